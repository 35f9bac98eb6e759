// Run-length segments of a flat batch, built on the device.
//
// The reference builds them on the host, request by request
// (src/loquetier_src/model_generation.py:267-283): consecutive requests with the same adapter id
// merge into one segment whose length is the sum of their token counts; `segment` is the running
// sum of the lengths, starting at 0.  Here the per-request arrays already live on the device
// (a scheduler that keeps its queues there never brings them back), so one workgroup scans them:
// a request opens a segment when it is the first one or its id differs from its predecessor's,
// the segment index is the running count of such requests, the first row the running sum of
// the lengths before it.
//
// The host cannot know the number of segments without waiting for the device, so every output
// has the capacity of the request count R: entries past the last segment describe empty segments
// (indptr = total rows, length 0, the last real adapter id), which every consumer of an indptr
// skips.  n_seg[0] and n_seg[1] receive the segment count and the row total.
#pragma once
#include "smlm_plan.hpp"

namespace smlm {

struct SegmentsArgs {
  const int32_t* req_adapter;  // [R]
  const int32_t* req_len;      // [R], negative lengths count as 0
  int32_t* seg_adapter;        // [R]
  int32_t* seg_len;            // [R]
  int32_t* seg_indptr;         // [R + 1]
  int32_t* n_seg;              // [2]: segments, rows
  int R;
};

__global__ __launch_bounds__(kPlanThreads) void segments_kernel(SegmentsArgs a) {
  __shared__ uint64_t wave_tot[17];
  __shared__ uint64_t carry_s;
  const int tid = threadIdx.x;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  // pass 1: segment starts.  low half of the scan counts opened segments, high half sums rows
  for (int base = 0; base < a.R; base += kPlanThreads) {
    const int i = base + tid;
    int id = 0, len = 0, open = 0;
    if (i < a.R) {
      id = a.req_adapter[i];
      len = a.req_len[i];
      len = len > 0 ? len : 0;
      open = i == 0 || a.req_adapter[i - 1] != id;
    }
    const uint64_t carry = carry_s;
    const uint64_t v = (uint64_t)(uint32_t)open | ((uint64_t)(uint32_t)len << 32);
    const uint64_t incl = block_scan_incl(v, wave_tot);
    const uint32_t seg = (uint32_t)incl + (uint32_t)carry - 1u;                       // this request's segment
    const uint32_t row = (uint32_t)(incl >> 32) + (uint32_t)(carry >> 32) - (uint32_t)len;  // its first row
    if (open) {
      a.seg_adapter[seg] = id;
      a.seg_indptr[seg] = (int32_t)row;
    }
    __syncthreads();  // everyone has read carry_s and wave_tot
    if (tid == 0) {
      const uint64_t t = wave_tot[16];
      carry_s = (uint64_t)((uint32_t)carry + (uint32_t)t) | ((uint64_t)((uint32_t)(carry >> 32) + (uint32_t)(t >> 32)) << 32);
    }
    __syncthreads();
  }
  const int S = (int)(uint32_t)carry_s, rows = (int)(uint32_t)(carry_s >> 32);
  const int last_id = a.R > 0 ? a.req_adapter[a.R - 1] : 0;
  // pass 2: the unused tail, then the lengths from the finished indptr
  for (int i = S + tid; i <= a.R; i += kPlanThreads) {
    a.seg_indptr[i] = rows;
    if (i < a.R) a.seg_adapter[i] = last_id;
  }
  if (tid == 0) a.n_seg[0] = S, a.n_seg[1] = rows;
  __threadfence_block();
  __syncthreads();
  for (int i = tid; i < a.R; i += kPlanThreads) a.seg_len[i] = a.seg_indptr[i + 1] - a.seg_indptr[i];
}

}  // namespace smlm
