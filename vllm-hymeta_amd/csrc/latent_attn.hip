// Latent attention around its matrix products: the norms of the two latents, the rotation of the shared key part and
// the paged write of (latent, rotated key part); the assembly of the queries that are multiplied with those rows.
// The attention itself is hymeta_sink_attention with one key/value head whose value lies inside its key row.
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kMaxRotPairs = 256;

// cos and sin of position * freq, times mag, for a pair that turns; (1, 0) for a pair that passes unchanged.  The angle
// is formed and brought into [-pi, pi] in double precision (a position of a million times a frequency near one keeps
// all its digits); the functions themselves are the fp32 ones on that remainder.
__device__ __forceinline__ void rotation_of(const double* freqs, int i, int turning, int pos, float mag, float* c, float* s) {
  constexpr double kTwoPi = 6.283185307179586476925286766559, kInvTwoPi = 0.15915494309189533576888376337251;
  *c = 1.f, *s = 0.f;
  if (i < turning) {
    const double ang = static_cast<double>(pos) * freqs[i];
    const float r = static_cast<float>(fma(-kTwoPi, rint(ang * kInvTwoPi), ang));
    *c = cosf(r) * mag;
    *s = sinf(r) * mag;
  }
}

__device__ __forceinline__ void fill_rotation(float* s_cos, float* s_sin, const double* freqs, int pairs, int turning, int pos, float mag) {
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) rotation_of(freqs, i, turning, pos, mag, &s_cos[i], &s_sin[i]);
}

// RMS norm of n columns by one wave: src -> dst (may be the same), times weight.  Up to 64 * kPrepPerLane columns are
// read once (a lane keeps its columns between the sum and the scaling).
constexpr int kPrepPerLane = 16;
template <typename A>
__device__ __forceinline__ void wave_rms_norm(const typename A::elem* src, typename A::elem* dst, const float* weight, int n, float eps, int lane) {
  float ss = 0.f;
  if (n <= 64 * kPrepPerLane) {
    float v[kPrepPerLane];
#pragma unroll
    for (int u = 0; u < kPrepPerLane; ++u) {
      const int c = lane + 64 * u;
      v[u] = c < n ? A::ld(src + c) : 0.f;
      ss = fmaf(v[u], v[u], ss);
    }
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(n) + eps);
#pragma unroll
    for (int u = 0; u < kPrepPerLane; ++u) {
      const int c = lane + 64 * u;
      if (c < n) A::st(dst + c, v[u] * inv * weight[c]);
    }
    return;
  }
  for (int c = lane; c < n; c += 64) {
    const float v = A::ld(src + c);
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(n) + eps);
  for (int c = lane; c < n; c += 64) A::st(dst + c, A::ld(src + c) * inv * weight[c]);
}

// grid = tokens in fours, a wave per token (no barrier: the statistics are wave sums).
template <typename A>
__global__ __launch_bounds__(256) void latent_kv_prep_kernel(hymeta_latent_kv_prep_args a) {
  typedef typename A::elem elem;
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= a.num_tokens) return;
  const int s = seq_of_row(a.query_start_loc, a.num_seqs, t);
  const int pos = max(a.seq_lens[s] - (a.query_start_loc[s + 1] - t), 0);
  elem* row = static_cast<elem*>(a.proj) + static_cast<int64_t>(t) * a.proj_stride_t;
  wave_rms_norm<A>(row + a.q_col, row + a.q_col, a.q_norm_weight, a.q_rank, a.eps, lane);         // the query latent, in place
  const int64_t slot = a.slot_mapping ? a.slot_mapping[t] : -1;
  if (slot < 0 || slot >= a.num_blocks * a.block_size || a.kv_cache == nullptr) return;
  elem* dst = static_cast<elem*>(a.kv_cache) + slot * static_cast<int64_t>(a.kv_rank + a.rot_dim);
  const elem* kv = row + a.kv_col;
  wave_rms_norm<A>(kv, dst, a.kv_norm_weight, a.kv_rank, a.eps, lane);
  for (int i = lane; i < a.rot_dim / 2; i += 64) {
    float c, sn;
    rotation_of(a.rot_freqs, i, a.rot_dims / 2, pos, a.rot_mag, &c, &sn);
    const float u = A::ld(kv + a.kv_rank + 2 * i), v = A::ld(kv + a.kv_rank + 2 * i + 1);
    A::st(dst + a.kv_rank + 2 * i, u * c - v * sn);
    A::st(dst + a.kv_rank + 2 * i + 1, v * c + u * sn);
  }
}

template <typename A>
__global__ __launch_bounds__(256) void latent_q_assemble_kernel(hymeta_latent_q_assemble_args a) {
  typedef typename A::elem elem;
  __shared__ float s_cos[kMaxRotPairs], s_sin[kMaxRotPairs];
  const int t = blockIdx.x;
  const int s = seq_of_row(a.query_start_loc, a.num_seqs, t);
  const int pos = a.seq_lens[s] - (a.query_start_loc[s + 1] - t);
  const int pairs = a.rot_dim / 2, C = a.kv_rank;
  fill_rotation(s_cos, s_sin, a.rot_freqs, pairs, a.rot_dims / 2, pos < 0 ? 0 : pos, a.rot_mag);
  __syncthreads();
  const elem* q = static_cast<const elem*>(a.q) + static_cast<int64_t>(t) * a.q_stride_t;
  elem* out = static_cast<elem*>(a.out) + static_cast<int64_t>(t) * a.num_heads * (C + a.rot_dim);
  // one element of the absorbed part, or one pair of the rotated part, per thread and round, over all heads at once
  const int per_head = C + pairs;
  for (int idx = threadIdx.x; idx < a.num_heads * per_head; idx += 256) {
    const int h = idx / per_head, j = idx % per_head;
    elem* o = out + static_cast<int64_t>(h) * (C + a.rot_dim);
    if (j < C) {
      o[j] = static_cast<const elem*>(a.q_abs)[(static_cast<int64_t>(h) * a.num_tokens + t) * C + j];
    } else {
      const int i = j - C;
      const elem* qr = q + static_cast<int64_t>(h) * (a.dim + a.rot_dim) + a.dim;
      const float u = A::ld(qr + 2 * i), v = A::ld(qr + 2 * i + 1);
      A::st(o + C + 2 * i, u * s_cos[i] - v * s_sin[i]);
      A::st(o + C + 2 * i + 1, v * s_cos[i] + u * s_sin[i]);
    }
  }
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_latent_kv_prep(const hymeta_latent_kv_prep_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_latent_kv_prep_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.q_rank <= 0 || a.kv_rank <= 0 || a.rot_dim < 0 || a.rot_dims < 0 || a.q_col < 0 ||
      a.kv_col < 0 || a.block_size <= 0 || a.num_blocks < 0)
    return HYMETA_ERR_INVALID_ARG;
  if (a.rot_dim % 2 != 0 || a.rot_dims % 2 != 0 || a.rot_dims > a.rot_dim) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.rot_dim / 2 > kMaxRotPairs) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.proj || !a.q_norm_weight || !a.kv_norm_weight || !a.query_start_loc || !a.seq_lens || (a.rot_dims > 0 && !a.rot_freqs))
    return HYMETA_ERR_INVALID_ARG;
  if (a.slot_mapping && !a.kv_cache) return HYMETA_ERR_INVALID_ARG;
  if (a.proj_stride_t < a.q_col + a.q_rank || a.proj_stride_t < a.kv_col + a.kv_rank + a.rot_dim) return HYMETA_ERR_INVALID_ARG;
  const bool apart = a.q_col + a.q_rank <= a.kv_col || a.kv_col + a.kv_rank + a.rot_dim <= a.q_col;
  if (!apart) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(latent_kv_prep_kernel<ActBf16>, dim3((a.num_tokens + 3) / 4), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(latent_kv_prep_kernel<ActF32>, dim3((a.num_tokens + 3) / 4), dim3(256), 0, st, a);
  return launch_status();
}

extern "C" int hymeta_latent_q_assemble(const hymeta_latent_q_assemble_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_latent_q_assemble_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.num_heads <= 0 || a.dim < 0 || a.rot_dim < 0 || a.rot_dims < 0 || a.kv_rank <= 0)
    return HYMETA_ERR_INVALID_ARG;
  if (a.rot_dim % 2 != 0 || a.rot_dims % 2 != 0 || a.rot_dims > a.rot_dim) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.rot_dim / 2 > kMaxRotPairs) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.q || !a.q_abs || !a.out || !a.query_start_loc || !a.seq_lens || (a.rot_dims > 0 && !a.rot_freqs)) return HYMETA_ERR_INVALID_ARG;
  if (a.q_stride_t < static_cast<int64_t>(a.num_heads) * (a.dim + a.rot_dim)) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(latent_q_assemble_kernel<ActBf16>, dim3(a.num_tokens), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(latent_q_assemble_kernel<ActF32>, dim3(a.num_tokens), dim3(256), 0, st, a);
  return launch_status();
}
