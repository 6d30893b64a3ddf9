// Linear attention with a constant decay per head ("lightning attention"): S <- decay S + k v^T, out = S^T q, the state
// fp32 and carried per sequence; and the output norm with its sigmoid gate.
#include "act_types.h"

namespace hymeta {

namespace {

__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }

// Token by token.  grid = (heads, sequences, value columns in runs of 256); a thread owns one value column c and keeps
// that column of the state, S[:, c], in registers; q_t and k_t go through LDS.
template <typename A, int DMAX>
__global__ __launch_bounds__(256) void lightning_rows_kernel(hymeta_lightning_attention_args a) {
  typedef typename A::elem elem;
  __shared__ float s_q[2][DMAX], s_k[2][DMAX];
  const int h = blockIdx.x, s = blockIdx.y;
  const int c = blockIdx.z * 256 + threadIdx.x;
  const int H = a.num_heads, D = a.head_dim, Dv = a.v_dim;
  const int r0 = a.query_start_loc[s], r1 = a.query_start_loc[s + 1];
  if (r1 <= r0) return;
  const int slot = a.slot_idx[s];
  const bool live = c < Dv;
  float* st = (slot >= 0) ? a.state + ((static_cast<int64_t>(slot) * H + h) * D) * Dv : nullptr;
  float S[DMAX];
  const bool carry = st != nullptr && a.context_lens[s] > 0 && live;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) S[d] = (carry && d < D) ? st[static_cast<int64_t>(d) * Dv + c] : 0.f;
  const float decay = a.decay[h];
  const int64_t q_off = static_cast<int64_t>(h) * D, k_off = static_cast<int64_t>(H) * D + q_off;
  const int64_t v_off = 2 * static_cast<int64_t>(H) * D + static_cast<int64_t>(h) * Dv;
  for (int t = r0; t < r1; ++t) {
    const elem* row = static_cast<const elem*>(a.qkv) + static_cast<int64_t>(t) * a.qkv_stride_t;
    const int buf = (t - r0) & 1;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
      s_q[buf][d] = silu_f(A::ld(row + q_off + d));
      s_k[buf][d] = silu_f(A::ld(row + k_off + d));
    }
    const float v = live ? silu_f(A::ld(row + v_off + c)) : 0.f;
    __syncthreads();           // one barrier per token: the next token fills the other buffer
    float o = 0.f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < D) {
        S[d] = fmaf(decay, S[d], s_k[buf][d] * v);
        o = fmaf(S[d], s_q[buf][d], o);
      }
    }
    if (live) a.out[static_cast<int64_t>(t) * H * Dv + static_cast<int64_t>(h) * Dv + c] = o;
  }
  if (st != nullptr && live) {
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
      if (d < D) st[static_cast<int64_t>(d) * Dv + c] = S[d];
  }
}

template <typename A>
__global__ __launch_bounds__(256) void gated_rms_norm_kernel(hymeta_gated_rms_norm_args a) {
  typedef typename A::elem elem;
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const float* x = a.x + t * a.width;
  const elem* g = static_cast<const elem*>(a.gate) + t * a.gate_stride_t;
  elem* out = static_cast<elem*>(a.out) + t * a.width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < a.width; c += 256) ss = fmaf(x[c], x[c], ss);
  ss = block_sum<4>(ss, red);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(a.width) + a.eps);
  for (int c = threadIdx.x; c < a.width; c += 256) A::st(out + c, x[c] * inv * a.weight[c] * sigmoid_exact(A::ld(g + c)));
}

template <typename A>
void launch_rows(const hymeta_lightning_attention_args& a, hipStream_t st) {
  const dim3 grid(a.num_heads, a.num_seqs, (a.v_dim + 255) / 256);
  const dim3 block(a.v_dim >= 256 ? 256 : (a.v_dim + 63) / 64 * 64);
  if (a.head_dim <= 32) hipLaunchKernelGGL((lightning_rows_kernel<A, 32>), grid, block, 0, st, a);
  else if (a.head_dim <= 64) hipLaunchKernelGGL((lightning_rows_kernel<A, 64>), grid, block, 0, st, a);
  else if (a.head_dim <= 128) hipLaunchKernelGGL((lightning_rows_kernel<A, 128>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((lightning_rows_kernel<A, 256>), grid, block, 0, st, a);
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_lightning_attention(const hymeta_lightning_attention_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_lightning_attention_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.num_heads <= 0 || a.head_dim <= 0 || a.v_dim <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.head_dim > 256 || a.num_seqs > 65535 || a.v_dim > 256 * 65535) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.qkv || !a.state || !a.decay || !a.out || !a.query_start_loc || !a.context_lens || !a.slot_idx) return HYMETA_ERR_INVALID_ARG;
  if (a.qkv_stride_t < static_cast<int64_t>(a.num_heads) * (2 * a.head_dim + a.v_dim)) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) launch_rows<ActBf16>(a, st);
  else launch_rows<ActF32>(a, st);
  return launch_status();
}

extern "C" int hymeta_gated_rms_norm(const hymeta_gated_rms_norm_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_gated_rms_norm_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.x || !a.gate || !a.weight || !a.out || a.gate_stride_t < a.width) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(gated_rms_norm_kernel<ActBf16>, dim3(a.num_tokens), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(gated_rms_norm_kernel<ActF32>, dim3(a.num_tokens), dim3(256), 0, st, a);
  return launch_status();
}
