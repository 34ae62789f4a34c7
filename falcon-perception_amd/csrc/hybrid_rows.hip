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
// That closed form equals the reference's mask exactly when every span opens and closes
// inside one document of the packed row (what the reference's engine packs,
// paged_inference.py:637-672: whole sequences, each padded to 128).  Two inputs break it and
// are reported through `status` instead of being answered wrongly:
//   bit 0  an eoi with no span open -- the chunk starts inside an image span whose soi lies in
//          an earlier chunk.  The caller can declare that with `open_at_start[slot] != 0`: the
//          first row of that slot's run then counts as preceded by a soi, and the rows up to
//          the eoi get the eoi's index as their limit (every earlier key of the span is below
//          the row anyway, so one limit per row still is the whole mask);
//   bit 1  a span still open where the document changes or the row ends -- its rows would need
//          keys of another document (what the reference's global counts would allow) or keys
//          that are not in the cache yet.
//
// One workgroup scans the packed row.  The tokens are first classified with loads that run over the row in
// memory order (two tokens per lane and step), four bits per token into LDS: how many soi it counts as (its own
// and a virtual one in front of a declared run), whether it is an eoi, whether its document ends after it.
// Then each thread owns a contiguous chunk of the classes: the chunk totals are combined with a prefix sum
// (forward) and a suffix minimum (backward), inside the wavefronts by lane shifts and over the 16 wavefront totals
// through LDS; the limits are staged in LDS and leave in memory order.  L is at most 65536 tokens; 23040 take 21
// microseconds and 32768 take 32 (reading the ids chunk by chunk, every lane at its own stride, took 61 for 23040).
#include "fp_common.h"

namespace {

constexpr int kThreads = 1024;
constexpr int kMaxL = 65536;
constexpr int kSoiMask = 3, kEoiBit = 4, kRunEndBit = 8;
constexpr int kSegment = 32768;  // rows whose limits are staged in LDS at a time (as limit - 1, 16 bits: a limit is 1 .. 65536)

__global__ __launch_bounds__(kThreads) void hybrid_row_limits_kernel(const int64_t* __restrict__ ids,
                                                                     const int64_t* __restrict__ docs,
                                                                     const uint8_t* __restrict__ open_at_start,
                                                                     int max_batch, int L,
                                                                     int64_t soi, int64_t eoi,
                                                                     int32_t* __restrict__ row_hi,
                                                                     int32_t* __restrict__ status) {
  __shared__ uint8_t s_cls[kMaxL / 2];  // two tokens per byte
  __shared__ int s_soi[kThreads / 64];
  __shared__ int s_eoi[kThreads / 64];
  __shared__ int s_next[kThreads / 64];
  __shared__ int s_flags;
  __shared__ uint16_t s_out[kSegment];

  const int tid = threadIdx.x;
  if (tid == 0) s_flags = 0;

  // class of token k; d_prev / d / d_next are the documents of k - 1, k, k + 1 (unused without docs)
  auto classify = [&](int k, int64_t id, int64_t d_prev, int64_t d, int64_t d_next) {
    int c = (id == soi) | ((id == eoi) ? kEoiBit : 0);
    if (docs) {
      // a soi counted in front of token k: k starts a run of a slot declared open
      if (open_at_start && (k == 0 || d_prev != d) && d >= 0 && d < max_batch && open_at_start[d] != 0) c += 1;
      if (k == L - 1 || d_next != d) c |= kRunEndBit;
    } else if (k == L - 1) {
      c |= kRunEndBit;
    }
    return c;
  };
  // kBatch steps of a lane at a time: every load of the batch is requested before the first class is computed
  // (step by step the loop was a chain of round trips to memory, a dozen of them at 23040 tokens)
  constexpr int kBatch = 4;
  for (int i0 = tid; 2 * i0 < L; i0 += kBatch * kThreads) {
    int64_t id0[kBatch], id1[kBatch], dm[kBatch], d0[kBatch], d1[kBatch], d2[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int k0 = 2 * (i0 + j * kThreads), k1 = k0 + 1;
      const bool one = k0 < L, two = k1 < L;
      id0[j] = one ? ids[k0] : 0;
      id1[j] = two ? ids[k1] : 0;
      dm[j] = d0[j] = d1[j] = d2[j] = 0;
      if (docs) {
        dm[j] = one && k0 > 0 ? docs[k0 - 1] : 0;
        d0[j] = one ? docs[k0] : 0;
        d1[j] = two ? docs[k1] : 0;
        d2[j] = k1 + 1 < L ? docs[k1 + 1] : 0;
      }
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int i = i0 + j * kThreads;
      const int k0 = 2 * i, k1 = k0 + 1;
      if (k0 >= L) break;
      int byte = classify(k0, id0[j], dm[j], d0[j], d1[j]);
      if (k1 < L) byte |= classify(k1, id1[j], d0[j], d1[j], d2[j]) << 4;
      s_cls[i] = static_cast<uint8_t>(byte);
    }
  }
  __syncthreads();
  auto cls = [&](int k) { return (s_cls[k >> 1] >> ((k & 1) * 4)) & 15; };

  const int per = (L + kThreads - 1) / kThreads;
  const int lo = min(tid * per, L);
  const int hi = min(lo + per, L);

  int n_soi = 0, n_eoi = 0;
  for (int k = lo; k < hi; ++k) {
    const int c = cls(k);
    n_soi += c & kSoiMask;
    n_eoi += (c & kEoiBit) != 0;
  }
  // inclusive prefix sums over the chunk totals: inside every wavefront by lane shifts, then over the 16
  // wavefront totals through LDS (two barriers instead of the twenty of a scan over all 1024 threads)
  const int lane = tid & 63, wave = tid >> 6;
  int inc_soi = n_soi, inc_eoi = n_eoi;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int a = __shfl_up(inc_soi, d), b = __shfl_up(inc_eoi, d);
    if (lane >= d) {
      inc_soi += a;
      inc_eoi += b;
    }
  }
  if (lane == 63) {
    s_soi[wave] = inc_soi;
    s_eoi[wave] = inc_eoi;
  }
  __syncthreads();
  for (int w = 0; w < wave; ++w) {
    inc_soi += s_soi[w];
    inc_eoi += s_eoi[w];
  }
  const int base_soi = inc_soi - n_soi;  // counts before this chunk
  const int base_eoi = inc_eoi - n_eoi;

  // first index in this chunk that ends a span (not inside, or a soi), L if none
  int first_end = L;
  int flags = 0;
  {
    int o = base_soi, c = base_eoi;
    for (int k = lo; k < hi; ++k) {
      const int cl = cls(k);
      o += cl & kSoiMask;
      c += (cl & kEoiBit) != 0;
      const bool ends = !(o - c > 0) || (cl & kSoiMask);
      if (ends && first_end == L) first_end = k;
      if (o - c < 0) flags |= 1;
      if ((cl & kRunEndBit) && o - c > 0) flags |= 2;
    }
  }
  if (flags) atomicOr(&s_flags, flags);
  // exclusive suffix minimum over chunks (the first span end after this chunk), the same way
  int suf = first_end;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int a = __shfl_down(suf, d);
    if (lane + d < 64) suf = min(suf, a);
  }
  if (lane == 0) s_next[wave] = suf;  // minimum of the whole wavefront
  __syncthreads();
  int next_end = __shfl_down(suf, 1);  // minimum over the later lanes of this wavefront
  if (lane == 63) next_end = L;
  for (int w = wave + 1; w < kThreads / 64; ++w) next_end = min(next_end, s_next[w]);

  // walk the chunk backwards; counts at k are recovered by undoing token k+1.  The limits go to global memory
  // through LDS, a segment of kSegment rows at a time from the last to the first: written from the chunks they
  // would leave as 4-byte pieces `per` rows apart, 64 different cache lines per store instruction.
  int o = base_soi + n_soi, c = base_eoi + n_eoi;  // inclusive counts at hi - 1
  int k = hi - 1;
  for (int seg_lo = ((L - 1) / kSegment) * kSegment; seg_lo >= 0; seg_lo -= kSegment) {
    for (; k >= lo && k >= seg_lo; --k) {
      const int cl = cls(k);
      const bool inside = o - c > 0;
      s_out[k - seg_lo] = static_cast<uint16_t>((inside ? next_end : k + 1) - 1);
      if (!inside || (cl & kSoiMask)) next_end = k;
      o -= cl & kSoiMask;
      c -= (cl & kEoiBit) != 0;
    }
    __syncthreads();
    const int n = min(kSegment, L - seg_lo);
    for (int i = tid; i < n; i += kThreads) row_hi[seg_lo + i] = static_cast<int>(s_out[i]) + 1;
    __syncthreads();
  }
  if (tid == 0 && status) *status = s_flags;  // every atomicOr lies before the barriers of the suffix scan
}

}  // namespace

extern "C" int fp_hybrid_row_limits(const int64_t* input_ids, const int64_t* batch_idx,
                                    const uint8_t* open_at_start, int32_t max_batch, int32_t L,
                                    int64_t soi_id, int64_t eoi_id, int32_t* row_hi, int32_t* status,
                                    void* stream) {
  if (L < 0) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_hybrid_row_limits: negative length");
  if (L > kMaxL) return fp::fail(FP_ERR_UNSUPPORTED, "fp_hybrid_row_limits: L=%d exceeds %d", L, kMaxL);
  if (L == 0) return FP_OK;
  if (!input_ids || !row_hi) return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_hybrid_row_limits: null pointer");
  if (open_at_start && (!batch_idx || max_batch <= 0))
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_hybrid_row_limits: open_at_start needs batch_idx and max_batch");
  hipLaunchKernelGGL(hybrid_row_limits_kernel, dim3(1), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                     input_ids, batch_idx, open_at_start, max_batch, L, soi_id, eoi_id, row_hi, status);
  return fp::check_launch("fp_hybrid_row_limits");
}
