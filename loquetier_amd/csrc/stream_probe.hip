// Plain streaming kernels of known traffic, for the benchmark only: what an HBM-bound launch of a
// given size reaches on this part.  Built into its own small library (libsmlm_probe.so); the
// operator library does not contain it.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define SMLM_GLOBAL __attribute__((address_space(1)))

// Every thread reads U 16-byte pieces a whole grid apart (all requested before the first is used)
// and, when WRITE, writes them back incremented: 16 bytes read (+ 16 written) per piece.
template <int U, bool WRITE>
__global__ __launch_bounds__(256) void stream_kernel(u32x4* p, size_t n16, uint32_t* sink) {
  const size_t stride = (size_t)gridDim.x * 256;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  u32x4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t j = i + u * stride;
    v[u] = __builtin_nontemporal_load((const SMLM_GLOBAL u32x4*)(p + (j < n16 ? j : 0)));
  }
  uint32_t acc = 0;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t j = i + u * stride;
    if (WRITE) {
      if (j < n16) __builtin_nontemporal_store(v[u] + 1u, (SMLM_GLOBAL u32x4*)(p + j));
    } else {
      acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    }
  }
  if (!WRITE && acc == 0x9e3779b9u && sink) *sink = acc;  // keeps the loads alive
}

extern "C" {

// read-modify-write of `bytes` bytes at p (moves 2 * bytes); returns 0 or -1
__attribute__((visibility("default"))) int smlm_probe_rmw(void* p, size_t bytes, void* stream) {
  const size_t n16 = bytes / 16;
  if (!p || !n16) return -1;
  const unsigned nb = (unsigned)((n16 + 256 * 8 - 1) / (256 * 8));
  stream_kernel<8, true><<<nb, 256, 0, (hipStream_t)stream>>>((u32x4*)p, n16, nullptr);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

// read of `bytes` bytes at p
__attribute__((visibility("default"))) int smlm_probe_read(void* p, size_t bytes, void* sink, void* stream) {
  const size_t n16 = bytes / 16;
  if (!p || !n16) return -1;
  const unsigned nb = (unsigned)((n16 + 256 * 8 - 1) / (256 * 8));
  stream_kernel<8, false><<<nb, 256, 0, (hipStream_t)stream>>>((u32x4*)p, n16, (uint32_t*)sink);
  return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // extern "C"
