// Activation element types of the kernels that run in bf16 or in fp32 (act_dtype of their argument
// structs): loads widen to fp32, stores round once.
#pragma once

#include "common.h"

namespace hymeta {

struct ActBf16 {
  typedef uint16_t elem;
  static constexpr int kDtype = HYMETA_BF16;
  static __device__ __forceinline__ float ld(const elem* p) { return bf2f(*p); }
  static __device__ __forceinline__ void st(elem* p, float v) { *p = f2bf(v); }
  static __device__ __forceinline__ float round(float v) { return bf16_round(v); }
  // four consecutive elements, 8-byte aligned
  static __device__ __forceinline__ void ld4(const elem* p, float* v) {
    const u32x2 t = *reinterpret_cast<const u32x2*>(p);
    v[0] = lo_bf(t[0]), v[1] = hi_bf(t[0]), v[2] = lo_bf(t[1]), v[3] = hi_bf(t[1]);
  }
  static __device__ __forceinline__ void st4(elem* p, const float* v) {
    *reinterpret_cast<u32x2*>(p) = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
  }
  // fp32 in, fp32 out, the hardware's exponential (about 2 ulp): where the inputs carry 8 bits
  static __device__ __forceinline__ float sigmoid(float x) { return 1.f / (1.f + __expf(-x)); }
};

struct ActF32 {
  typedef float elem;
  static constexpr int kDtype = HYMETA_F32;
  static __device__ __forceinline__ float ld(const elem* p) { return *p; }
  static __device__ __forceinline__ void st(elem* p, float v) { *p = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
  // four consecutive elements, 16-byte aligned
  static __device__ __forceinline__ void ld4(const elem* p, float* v) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p);
    v[0] = t[0], v[1] = t[1], v[2] = t[2], v[3] = t[3];
  }
  static __device__ __forceinline__ void st4(elem* p, const float* v) { *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]}; }
  static __device__ __forceinline__ float sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
};

inline bool act_dtype_ok(int d) { return d == HYMETA_BF16 || d == HYMETA_F32; }

// Sum over the 64 lanes of a wave, result in every lane.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Sum over a workgroup of `Waves` waves; `red` is Waves floats of LDS.  Every thread gets the sum.  The
// summation order is fixed (lanes by butterfly, waves in order), so a row's statistic does not depend
// on which workgroup computes it.
template <int Waves>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();                       // red may still be read from the call before
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < Waves; ++w) s += red[w];
  return s;
}

// Sequence of a token row: the s with query_start_loc[s] <= t < query_start_loc[s + 1].
__device__ __forceinline__ int seq_of_row(const int32_t* query_start_loc, int num_seqs, int t) {
  int lo = 0, hi = num_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (query_start_loc[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ float sigmoid_exact(float x) { return 1.f / (1.f + expf(-x)); }

}  // namespace hymeta
