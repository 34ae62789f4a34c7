// Shared helpers of the gfx950 kernels behind include/fp_paged_kv.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "fp_paged_kv.h"

namespace fp {

// thread-local message of the last failing entry point
char* error_buffer();
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

inline int elem_bytes(int dtype) {
  switch (dtype) {
    case FP_DTYPE_F32: return 4;
    case FP_DTYPE_BF16: return 2;
    case FP_DTYPE_F16: return 2;
    default: return 0;
  }
}

// CUs of the current device (asked once per device; the answer never changes)
int compute_units();

inline bool aligned(const void* p, int n) { return (reinterpret_cast<uintptr_t>(p) % n) == 0; }

// log2 of x if x is a power of two, else -1
inline int log2_exact(int x) {
  if (x <= 0 || (x & (x - 1))) return -1;
  int s = 0;
  while ((1 << s) < x) ++s;
  return s;
}

// position / length arrays come as int32 (decode) or int64 (prefill)
__device__ __forceinline__ int64_t load_index(const void* p, int64_t i, int is_i64) {
  return is_i64 ? static_cast<const int64_t*>(p)[i] : static_cast<int64_t>(static_cast<const int32_t*>(p)[i]);
}

// t / P and t % P with the shift fast path for power-of-two page sizes
struct PageDiv {
  int page_size;
  int shift;  // >= 0 when page_size is a power of two
  __host__ explicit PageDiv(int p) : page_size(p), shift(log2_exact(p)) {}
  __device__ __forceinline__ void split(int64_t t, int64_t& blk, int& off) const {
    if (shift >= 0) {
      blk = t >> shift;
      off = static_cast<int>(t & (page_size - 1));
    } else {
      blk = t / page_size;
      off = static_cast<int>(t - blk * page_size);
    }
  }
};

// fp32 chunked-prefill attention on the fp32 matrix instruction (paged_prefill_f32.hip)
int prefill_mfma_f32(const void* q, int64_t q_stride_row, int64_t q_stride_h, const void* pool_k, const void* pool_v,
                     const int64_t* page_table, int64_t pt_row_stride, const int64_t* batch_idx,
                     const int32_t* row_limit, void* out, int64_t out_stride_row, int64_t out_stride_h, float* lse,
                     const float* sinks, int32_t Lq, int32_t Hq, int32_t Hc, int32_t D, int32_t page_size,
                     int32_t n_pages, int32_t max_batch, int64_t n_slots, float scale, void* workspace,
                     int64_t workspace_bytes, hipStream_t st);

// Key shares the prefill kernel of `dtype` cuts a launch of `wgs` workgroups into on the current device
// (1 .. 8), and the workspace bytes `shares` of them need (paged_prefill.hip)
int prefill_key_shares(int64_t wgs, int dtype);
int64_t prefill_share_bytes(int shares, int Lq, int Hq, int D, int elem_bytes);

}  // namespace fp
