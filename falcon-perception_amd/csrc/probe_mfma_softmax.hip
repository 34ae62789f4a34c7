// A measuring kernel, not part of the attention path: how well does a SIMD of this GPU overlap the matrix
// instructions of one 64-key tile of the bf16 prefill kernel with the softmax arithmetic of another?
//
// A "slot" is what one wavefront of paged_prefill_kernel does per 64-key tile at head_dim 128 on its 32 query
// rows with a declared score bound: 32 v_mfma_f32_32x32x16_bf16 (16 for O^T += V^T P^T, 16 for S^T = K Q^T, the K
// and V operands read from LDS) and, on the 32 scores a lane holds, 32 exp2, 32 additions for the row sum and
// 16 packs to bf16.  Nothing else: no staging loads, no barrier, no mask, no addresses.  Every wavefront runs
// `iters` x 2 slots, the matrix part and the vector part strictly in turn as the data dependencies of one
// query block demand; with several wavefronts per SIMD the hardware is free to run the matrix part of one
// beside the vector part of another, which is all the prefill kernel's schedule can hope for.
#include "fp_common.h"

#include <hip/hip_bf16.h>

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  bf16x2 v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
  return __builtin_bit_cast(uint32_t, v);
}

struct Block {
  f32x16 o[4];  // O^T accumulators: head_dim 128 x 32 query rows
  f32x16 s[2];  // S^T: 64 keys x 32 query rows
  u32x4 p[4];   // P^T as bf16: the B operand of the four key steps of V^T P^T
  u32x4 q[8];   // Q^T as bf16: the B operand of the eight head_dim steps of K Q^T
  float sum;
};

// O^T += V^T P^T (16 matrix instructions), then S^T = K Q^T (16); A operands from LDS, 16 bytes per lane each
template <bool kFresh>
__device__ __forceinline__ void matrix_part(Block& x, const u32x4* lds_v, const u32x4* lds_k) {
#pragma unroll
  for (int ks = 0; ks < 4; ++ks)
#pragma unroll
    for (int d = 0; d < 4; ++d) x.o[d] = mfma(lds_v[(ks * 4 + d) * 64], x.p[ks], x.o[d]);
  if (kFresh) {
    const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    x.s[0] = zero;
    x.s[1] = zero;
  }
#pragma unroll
  for (int ds = 0; ds < 8; ++ds)
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) x.s[kb] = mfma(lds_k[(ds * 2 + kb) * 64], x.q[ds], x.s[kb]);
}

// p = exp2(s) referred to a fixed point, row sum, pack to bf16
__device__ __forceinline__ void vector_part(Block& x) {
  float acc = 0.f;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 16; i += 2) {
      const float e0 = __builtin_amdgcn_exp2f(x.s[kb][i]);
      const float e1 = __builtin_amdgcn_exp2f(x.s[kb][i + 1]);
      acc += e0;
      acc += e1;
      const int w = kb * 8 + i / 2;
      x.p[w >> 2][w & 3] = pack2(e0, e1);
    }
  x.sum += acc;
}

constexpr int kModeMatrix = 0, kModeVector = 1, kModeBoth = 2;

template <int kMode, int kThreads>
__global__ __launch_bounds__(kThreads, 1) void probe_kernel(float* out, int iters) {
  __shared__ u32x4 tiles[2][2][16 * 64];  // [buffer][K or V][operand][lane]: 64 KB, as the kernel's double buffers
  const int lane = threadIdx.x & 63;
  Block x;
  const float seed = 1e-3f * static_cast<float>(lane + 1);
  u32x4 init[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    init[i] = u32x4{pack2(seed, 1.f), pack2(0.5f, seed), pack2(seed, seed), pack2(0.25f, 0.125f)} + static_cast<uint32_t>(i);
#pragma unroll
  for (int i = 0; i < 8; ++i) x.q[i] = init[i & 3] + 3u * i + (threadIdx.x >> 6);
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int i = 0; i < 16; ++i) x.o[d][i] = 0.f;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 16; ++i) x.s[kb][i] = seed;
#pragma unroll
  for (int i = 0; i < 4; ++i) x.p[i] = init[i];
  x.sum = 0.f;
  for (int i = threadIdx.x; i < 2 * 2 * 16 * 64; i += kThreads) (&tiles[0][0][0])[i] = init[i & 3] + static_cast<uint32_t>(i);
  __syncthreads();

  for (int it = 0; it < iters; ++it) {
    const u32x4* lds_v = &tiles[it & 1][1][lane];
    const u32x4* lds_k = &tiles[it & 1][0][lane];
#pragma unroll
    for (int slot = 0; slot < 2; ++slot) {
      if (kMode != kModeVector) {
        matrix_part<kMode == kModeBoth>(x, lds_v, lds_k);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (kMode != kModeMatrix) {
        if (kMode == kModeVector) {
          // the scores count as new every slot (no instruction): the exponentials are not hoisted out of the loop
          asm volatile("" : "+v"(x.s[0]), "+v"(x.s[1]));
        }
        vector_part(x);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  float r = x.sum;
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int i = 0; i < 16; ++i) r += x.o[d][i];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int i = 0; i < 16; ++i) r += x.s[kb][i];
  r += __builtin_bit_cast(float, x.p[0][0] ^ x.p[1][1] ^ x.p[2][2] ^ x.p[3][3]);
  out[static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x] = r;
}

template <int kMode>
int launch_mode(int waves_per_simd, int workgroups, int iters, float* out, hipStream_t st) {
  switch (waves_per_simd) {
    case 1: hipLaunchKernelGGL((probe_kernel<kMode, 256>), dim3(workgroups), dim3(256), 0, st, out, iters); return FP_OK;
    case 2: hipLaunchKernelGGL((probe_kernel<kMode, 512>), dim3(workgroups), dim3(512), 0, st, out, iters); return FP_OK;
    case 3: hipLaunchKernelGGL((probe_kernel<kMode, 768>), dim3(workgroups), dim3(768), 0, st, out, iters); return FP_OK;
    default: return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_probe_mfma_softmax: waves_per_simd = %d (1 .. 3: with four the kernel would spill registers)", waves_per_simd);
  }
}

}  // namespace

extern "C" int fp_probe_mfma_softmax(int mode, int waves_per_simd, int workgroups, int iters, float* out,
                                     int64_t out_floats, void* stream) {
  if (workgroups <= 0 || iters < 0 || !out)
    return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_probe_mfma_softmax: bad argument");
  if (out_floats < static_cast<int64_t>(workgroups) * 256 * waves_per_simd)
    return fp::fail(FP_ERR_WORKSPACE, "fp_probe_mfma_softmax: out needs one float per launched thread");
  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc;
  switch (mode) {
    case kModeMatrix: rc = launch_mode<kModeMatrix>(waves_per_simd, workgroups, iters, out, st); break;
    case kModeVector: rc = launch_mode<kModeVector>(waves_per_simd, workgroups, iters, out, st); break;
    case kModeBoth: rc = launch_mode<kModeBoth>(waves_per_simd, workgroups, iters, out, st); break;
    default: return fp::fail(FP_ERR_INVALID_ARGUMENT, "fp_probe_mfma_softmax: mode = %d (0 matrix, 1 vector, 2 both)", mode);
  }
  if (rc != FP_OK) return rc;
  return fp::check_launch("fp_probe_mfma_softmax");
}
