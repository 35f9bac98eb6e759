"""Pins of the dropout oracle (oracle/dropout_oracle.c): the generator against
the published known-answer vectors, the mask against what an iid Bernoulli mask
must satisfy, the values against torch's own arithmetic."""
import numpy as np
import pytest
import torch

# Random123 distribution, kat_vectors: philox4x32, 10 rounds: counter, key, result
PHILOX_KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
    ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
    ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
     [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
]


@pytest.mark.parametrize("ctr,key,want", PHILOX_KAT)
def test_philox_known_answers(oracle, ctr, key, want):
    assert oracle.philox4x32_10(ctr, key) == want


def test_mask_layout_follows_the_generator(oracle):
    """Element (t, j) is decided by 16-bit piece j % 8 of the block with counter
    (t, j / 8, offset) and key seed -- checked against the generator itself."""
    seed, offset, p = 0x123456789abcdef, 0xfedcba9876543210, 0.3
    keep = oracle.dropout_mask(5, 32, np.full(5, p, np.float32), seed, offset, row0=11)
    thresh = int(np.float32(p) * np.float32(65536.0))
    for t in range(5):
        for cb in range(4):
            w = oracle.philox4x32_10([11 + t, cb, offset & 0xffffffff, offset >> 32],
                                     [seed & 0xffffffff, seed >> 32])
            pieces = [(w[e >> 1] >> (16 * (e & 1))) & 0xffff for e in range(8)]
            assert keep[t, 8 * cb:8 * cb + 8].tolist() == [int(q >= thresh) for q in pieces]


@pytest.mark.parametrize("p", [0.05, 0.1, 0.5, 0.9])
def test_mask_is_bernoulli(oracle, p):
    rows, cols = 512, 2048
    keep = oracle.dropout_mask(rows, cols, np.full(rows, p, np.float32), 99, 3).astype(np.float64)
    q = 1.0 - int(np.float32(p) * 65536) / 65536.0   # kept probability after quantising p to 1/65536
    n = rows * cols
    assert abs(keep.mean() - q) < 5 * np.sqrt(q * (1 - q) / n)
    # per row and per column: no row or column is systematically favoured
    z_rows = (keep.mean(1) - q) / np.sqrt(q * (1 - q) / cols)
    z_cols = (keep.mean(0) - q) / np.sqrt(q * (1 - q) / rows)
    assert np.abs(z_rows).max() < 5.5 and np.abs(z_cols).max() < 5.5
    assert abs(z_rows.std() - 1) < 0.15 and abs(z_cols.std() - 1) < 0.1
    # neighbours are uncorrelated (within a block of eight, across blocks, across rows)
    for a, b in ((keep[:, :-1], keep[:, 1:]), (keep[:, :-8], keep[:, 8:]), (keep[:-1], keep[1:])):
        corr = ((a - q) * (b - q)).mean() / (q * (1 - q))
        assert abs(corr) < 5 / np.sqrt(a.size)


def test_pieces_are_uniform(oracle):
    """The 16-bit pieces behind the mask: chi-square over 256 bins of the value at which
    each element would start being kept."""
    rows, cols = 256, 1024
    # keep count as a function of p scans the distribution of the pieces: take bins by thresholds
    counts = []
    for k in range(0, 257, 16):
        p = np.float32(k / 256.0)
        m = oracle.dropout_mask(rows, cols, np.full(rows, min(p, 0.99999), np.float32), 5, 5)
        counts.append(rows * cols - int(m.sum()))   # dropped = pieces below the threshold
    diffs = np.diff(np.array(counts[:-1], np.float64))  # 15 equal-width bins
    expect = rows * cols / 16.0
    chi2 = ((diffs - expect) ** 2 / expect).sum()
    assert chi2 < 45.0   # 14 degrees of freedom: P(chi2 > 45) < 1e-4


def test_different_streams_are_independent(oracle):
    rows, cols, p = 256, 1024, 0.3
    rp = np.full(rows, p, np.float32)
    base = oracle.dropout_mask(rows, cols, rp, 1, 1)
    q = 1.0 - int(np.float32(p) * 65536) / 65536.0
    agree_iid = q * q + (1 - q) * (1 - q)
    for other in (oracle.dropout_mask(rows, cols, rp, 1, 2), oracle.dropout_mask(rows, cols, rp, 2, 1),
                  oracle.dropout_mask(rows, cols, rp, 1, 1 << 32), oracle.dropout_mask(rows, cols, rp, 1 << 32, 1),
                  oracle.dropout_mask(rows, cols, rp, 1, 1, row0=rows)):
        agree = (base == other).mean()
        assert abs(agree - agree_iid) < 5 * np.sqrt(agree_iid * (1 - agree_iid) / base.size)
    assert np.array_equal(base, oracle.dropout_mask(rows, cols, rp, 1, 1))            # reproducible
    assert np.array_equal(base[7:], oracle.dropout_mask(rows - 7, cols, rp[7:], 1, 1, row0=7))  # rows by absolute index


@pytest.mark.parametrize("dt,tdt", [("fp16", torch.float16), ("bf16", torch.bfloat16)])
def test_kept_values_match_torch_arithmetic(oracle, dt, tdt):
    rng = np.random.default_rng(3)
    rows, cols = 24, 256
    x = oracle.round_to(rng.standard_normal((rows, cols)).astype(np.float32) * 3, dt)
    row_p = np.array([0.0, 0.05, 0.1, 0.25, 0.5, 0.75] * 4, np.float32)
    out = oracle.dropout_rows(x, row_p, 17, 4, dt)
    keep = oracle.dropout_mask(rows, cols, row_p, 17, 4).astype(bool)
    for t in range(rows):
        xt = torch.from_numpy(x[t]).to(tdt)
        if row_p[t] == 0:
            want = xt.float().numpy()
            assert keep[t].all()
        else:
            # torch's dropout arithmetic: float product with the float factor, cast to the dtype
            scale = torch.tensor(1.0, dtype=torch.float32) / (1.0 - torch.tensor(row_p[t]))
            want = (xt.float() * scale).to(tdt).float().numpy() * keep[t]
        assert np.array_equal(out[t], want)


def test_limits_and_mean(oracle):
    rng = np.random.default_rng(4)
    x = oracle.round_to(rng.standard_normal((8, 64)).astype(np.float32), "bf16")
    assert np.array_equal(oracle.dropout_rows(x, np.zeros(8, np.float32), 1, 1, "bf16"), x)
    assert not oracle.dropout_rows(x, np.ones(8, np.float32), 1, 1, "bf16").any()  # torch: p = 1 gives zeros
    # E[dropout(x)] = x: average over many independent masks
    ones = np.ones((8, 64), np.float32)
    acc = np.zeros_like(ones, dtype=np.float64)
    n = 400
    for i in range(n):
        acc += oracle.dropout_rows(ones, np.full(8, 0.25, np.float32), 7, i, "fp32")
    assert abs(acc.mean() / n - 1.0) < 0.01
    # the functional form against torch's own dropout on a mask-independent statistic:
    # kept values are exactly x / (1 - p), so the set of output values is {0, x / (1 - p)}
    t = torch.nn.functional.dropout(torch.ones(4096), p=0.25, training=True)
    ours = oracle.dropout_rows(np.ones((1, 4096), np.float32), np.array([0.25], np.float32), 1, 1, "fp32")
    assert set(np.unique(ours)) == set(np.unique(t.numpy()))
