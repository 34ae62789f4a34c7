// Per-row key limits of the hybrid prefill mask, in closed form.
//
// The reference evaluates `image_prefix OR document-causal` on a dense [L, L] grid
// through a compiled create_block_mask on every prefill step
// (paged_attention.py:343-362, attention.py:75-96).  With
//   opened[k] = #soi tokens in ids[0..k],  closed[k] = #eoi tokens in ids[0..k],
//   inside[k] = opened[k] - closed[k] > 0,  span[k] = opened[k] * inside[k]
// the image-prefix set of an inside row q is the contiguous run of inside tokens
// with q's span id, which ends at the first k > q that is not inside or is a soi.
// So row q may see keys up to  row_hi[q] = inside[q] ? that k : q + 1.
//
// One workgroup scans the packed row: each thread owns a contiguous chunk, the
// chunk totals are combined with an LDS prefix sum (forward) and an LDS suffix
// minimum (backward).  L is at most 65536 tokens, the work is a few microseconds.
#include "fp_common.h"

namespace {

constexpr int kThreads = 1024;
constexpr int kMaxL = 65536;

__global__ __launch_bounds__(kThreads) void hybrid_row_limits_kernel(const int64_t* __restrict__ ids, int L,
                                                                     int64_t soi, int64_t eoi,
                                                                     int32_t* __restrict__ row_hi) {
  __shared__ int s_soi[kThreads];
  __shared__ int s_eoi[kThreads];
  __shared__ int s_next[kThreads];

  const int tid = threadIdx.x;
  const int per = (L + kThreads - 1) / kThreads;
  const int lo = min(tid * per, L);
  const int hi = min(lo + per, L);

  int n_soi = 0, n_eoi = 0;
  for (int k = lo; k < hi; ++k) {
    const int64_t id = ids[k];
    n_soi += id == soi;
    n_eoi += id == eoi;
  }
  s_soi[tid] = n_soi;
  s_eoi[tid] = n_eoi;
  __syncthreads();
  // inclusive prefix sums over the chunk totals
  for (int d = 1; d < kThreads; d <<= 1) {
    const int a = tid >= d ? s_soi[tid - d] : 0;
    const int b = tid >= d ? s_eoi[tid - d] : 0;
    __syncthreads();
    s_soi[tid] += a;
    s_eoi[tid] += b;
    __syncthreads();
  }
  const int base_soi = s_soi[tid] - n_soi;  // counts before this chunk
  const int base_eoi = s_eoi[tid] - n_eoi;

  // first index in this chunk that ends a span (not inside, or a soi), L if none
  int first_end = L;
  {
    int o = base_soi, c = base_eoi;
    for (int k = lo; k < hi; ++k) {
      const int64_t id = ids[k];
      o += id == soi;
      c += id == eoi;
      const bool ends = !(o - c > 0) || id == soi;
      if (ends && first_end == L) first_end = k;
    }
  }
  s_next[tid] = first_end;
  __syncthreads();
  // inclusive suffix minimum over chunks
  for (int d = 1; d < kThreads; d <<= 1) {
    const int a = tid + d < kThreads ? s_next[tid + d] : L;
    __syncthreads();
    s_next[tid] = min(s_next[tid], a);
    __syncthreads();
  }
  int next_end = tid + 1 < kThreads ? s_next[tid + 1] : L;  // first span end after this chunk

  // walk the chunk backwards; counts at k are recovered by undoing token k+1
  int o = base_soi + n_soi, c = base_eoi + n_eoi;  // inclusive counts at hi - 1
  for (int k = hi - 1; k >= lo; --k) {
    const int64_t id = ids[k];
    const bool inside = o - c > 0;
    row_hi[k] = inside ? next_end : k + 1;
    if (!inside || id == soi) next_end = k;
    o -= id == soi;
    c -= id == eoi;
  }
}

}  // namespace

extern "C" int fp_hybrid_row_limits(const int64_t* input_ids, int32_t L, int64_t soi_id, int64_t eoi_id,
                                    int32_t* row_hi, void* stream) {
  if (L < 0) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_hybrid_row_limits: negative length");
  if (L > kMaxL) return fp::fail(FP_ERR_UNSUPPORTED, "fp_hybrid_row_limits: L=%d exceeds %d", L, kMaxL);
  if (L == 0) return FP_OK;
  if (!input_ids || !row_hi) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_hybrid_row_limits: null pointer");
  hipLaunchKernelGGL(hybrid_row_limits_kernel, dim3(1), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                     input_ids, L, soi_id, eoi_id, row_hi);
  return fp::check_launch("fp_hybrid_row_limits");
}
