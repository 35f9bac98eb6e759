/*
 * CPU oracle for the dropout that the reference applies to the training rows of x
 * before the LoRA term (src/loquetier_src/models/mixed_lora.py:185-192:
 * `self.adapters[idx].dropout(x[start:end, :])`, an nn.Dropout(p) in training mode,
 * one p per adapter).
 *
 * TEST INFRASTRUCTURE ONLY: linked into oracle/_build/libsmlm_oracle.so, used by
 * tests/ only; never by the package.
 *
 * nn.Dropout's contract is: every element is kept independently with probability
 * 1 - p; kept elements are multiplied by 1 / (1 - p) in float and rounded to the
 * tensor's dtype; dropped elements become 0.  Which elements are kept comes from
 * torch's generator state and is not part of the contract, so the mask here is
 * defined by a counter-based generator instead (Philox4x32-10, Salmon et al., SC'11,
 * the generator family torch's own device dropout draws from): the eight 16-bit
 * pieces of
 *     philox4x32_10(counter = (row, col / 8, offset_lo, offset_hi), key = (seed_lo, seed_hi))
 * decide the eight elements col..col+7 of a row (piece e = bits 16(e%2).. of word
 * e/2); an element is dropped when its piece is below floor(p * 65536).  The same
 * (seed, offset) gives the same mask in the forward and in the backward.
 *
 * What is pinned and by what (tests/test_dropout_oracle.py):
 *   - the generator : the three known-answer vectors of the Random123 distribution
 *                     for philox4x32 with 10 rounds;
 *   - the mask      : kept fraction within binomial bounds of 1 - p, per row and per
 *                     column; chi-square uniformity of the 16-bit pieces; different
 *                     offsets / seeds / rows give masks that agree on a fraction
 *                     (1-p)^2 + p^2 of the elements, as independent masks do;
 *   - the values    : kept elements equal torch's x.float() * (1 / (1 - p)) cast to
 *                     the dtype; p = 0 is the identity; p = 1 zeroes everything
 *                     (torch's special case); E[out] = x.
 * Parity unpinned: the reference's actual mask bits (torch RNG state; no generator
 * here can reproduce them, and no reference test fixes them).
 *
 * dtype codes as in smlm_oracle.c: 0 = fp32 (no rounding), 1 = fp16, 2 = bf16.
 */
#include <stdint.h>
#include <stddef.h>

#define ORACLE_API __attribute__((visibility("default")))

void oracle_round(float* a, size_t n, int dtype); /* smlm_oracle.c */

ORACLE_API void oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
  for (int i = 0; i < 10; ++i) {
    if (i) {
      k0 += 0x9E3779B9u;
      k1 += 0xBB67AE85u;
    }
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
  }
  out[0] = c0, out[1] = c1, out[2] = c2, out[3] = c3;
}

/* threshold of the 16-bit pieces and the float factor of kept elements */
static void drop_params(float p, uint32_t* thresh, float* scale) {
  if (!(p > 0.0f)) {
    *thresh = 0, *scale = 1.0f;
  } else if (p >= 1.0f) {
    *thresh = 65536u, *scale = 0.0f;
  } else {
    *thresh = (uint32_t)(p * 65536.0f);
    *scale = 1.0f / (1.0f - p);
  }
}

/*
 * keep[t, j] (1 = kept) for rows row0 .. row0 + rows - 1 of the batch; row_p[t] is the
 * dropout probability of row t's adapter (0 = no dropout on that row).
 */
ORACLE_API int oracle_dropout_mask(uint8_t* keep, int rows, int cols, int row0, const float* row_p,
                                   uint64_t seed, uint64_t offset) {
  if (rows < 0 || cols < 0 || (cols & 7)) return -1;
  const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  for (int t = 0; t < rows; ++t) {
    uint32_t thresh;
    float scale;
    drop_params(row_p[t], &thresh, &scale);
    for (int cb = 0; cb < cols / 8; ++cb) {
      const uint32_t ctr[4] = {(uint32_t)(row0 + t), (uint32_t)cb, (uint32_t)offset, (uint32_t)(offset >> 32)};
      uint32_t w[4];
      oracle_philox4x32_10(ctr, key, w);
      for (int e = 0; e < 8; ++e) {
        const uint32_t piece = (w[e >> 1] >> (16 * (e & 1))) & 0xffffu;
        keep[(size_t)t * cols + 8 * cb + e] = piece >= thresh;
      }
    }
  }
  return 0;
}

/* out = dropout(x): kept -> round(x * scale), dropped -> +0.  out may alias x. */
ORACLE_API int oracle_dropout_rows(float* out, const float* x, int rows, int cols, int row0,
                                   const float* row_p, uint64_t seed, uint64_t offset, int dtype) {
  if (rows < 0 || cols < 0 || (cols & 7)) return -1;
  const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  for (int t = 0; t < rows; ++t) {
    uint32_t thresh;
    float scale;
    drop_params(row_p[t], &thresh, &scale);
    const int active = row_p[t] > 0.0f;
    for (int cb = 0; cb < cols / 8; ++cb) {
      const uint32_t ctr[4] = {(uint32_t)(row0 + t), (uint32_t)cb, (uint32_t)offset, (uint32_t)(offset >> 32)};
      uint32_t w[4];
      oracle_philox4x32_10(ctr, key, w);
      for (int e = 0; e < 8; ++e) {
        const size_t i = (size_t)t * cols + 8 * cb + e;
        const uint32_t piece = (w[e >> 1] >> (16 * (e & 1))) & 0xffffu;
        if (!active) {
          out[i] = x[i];
        } else if (piece >= thresh) {
          float v = x[i] * scale;
          oracle_round(&v, 1, dtype);
          out[i] = v;
        } else {
          out[i] = 0.0f;
        }
      }
    }
  }
  return 0;
}
