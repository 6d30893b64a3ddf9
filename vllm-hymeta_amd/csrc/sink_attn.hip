// Causal paged attention with a distance bias and a sink, for any head size, fp32 or bf16 rows:
// the per-head query / key norm with the paged key / value write, and the attention itself.
//
// Scores, the running maximum, the weights and the weighted sum of the values are fp32 whatever the
// activation type.  The sink is a key of score 0 without a value: the running maximum starts at 0
// and the denominator at exp(0 - 0) = 1, everything else is the ordinary streaming softmax.
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kMaxHeadDim = 512;
constexpr int kMaxVChunks = 4;       // value size <= 256

// grid = tokens; a wave per (token, head) task: query heads, then key heads, then value heads.
template <typename A>
__global__ __launch_bounds__(256) void qk_norm_cache_kernel(hymeta_qk_norm_cache_args a) {
  typedef typename A::elem elem;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int H = a.num_heads, G = a.num_kv_heads, D = a.head_dim, Dv = a.v_dim;
  elem* row = static_cast<elem*>(a.qkv) + t * a.qkv_stride_t;
  const int64_t slot = a.slot_mapping ? a.slot_mapping[t] : -1;
  const bool store = slot >= 0 && slot < a.num_blocks * a.block_size;
  elem* cache = static_cast<elem*>(a.kv_cache) + (store ? slot : 0) * G * static_cast<int64_t>(D + Dv);
  for (int task = wave; task < H + 2 * G; task += 4) {
    if (task < H + G) {
      const bool is_q = task < H;
      elem* src = row + static_cast<int64_t>(task) * D;          // q heads, then k heads, contiguous
      const float* w = is_q ? a.q_weight : a.k_weight;
      if (!is_q && !store && w == nullptr) continue;
      float inv = 1.f;
      if (w != nullptr) {
        float ss = 0.f;
        for (int d = lane; d < D; d += 64) {
          const float v = A::ld(src + d);
          ss += v * v;
        }
        ss = wave_sum(ss);
        inv = 1.f / sqrtf(ss / static_cast<float>(D) + a.eps);
      }
      elem* dst = is_q ? src : cache + static_cast<int64_t>(task - H) * (D + Dv);
      if (is_q && w == nullptr) continue;
      if (!is_q && !store) continue;
      for (int d = lane; d < D; d += 64) {
        const float v = A::ld(src + d);
        A::st(dst + d, w ? v * inv * w[d] : v);
      }
    } else if (store) {
      const int g = task - H - G;
      const elem* src = row + static_cast<int64_t>(H + G) * D + static_cast<int64_t>(g) * Dv;
      elem* dst = cache + static_cast<int64_t>(g) * (D + Dv) + D;
      for (int d = lane; d < Dv; d += 64) dst[d] = src[d];
    }
  }
}

__device__ __forceinline__ float distance_bias(int mode, float a, float b, int dist) {
  return mode == HYMETA_BIAS_LOG_DISTANCE ? a * log1pf(b * static_cast<float>(dist)) : 0.f;
}

// One wave per (query row, head).  Keys in tiles of 64: lane = key for the scores, lane = value channel for the
// weighted sum, the tile's weights and row addresses handed over through LDS.
template <typename A>
__global__ __launch_bounds__(64) void sink_attention_rows_kernel(hymeta_sink_attention_args a) {
  typedef typename A::elem elem;
  __shared__ float s_q[kMaxHeadDim];
  __shared__ float s_p[64];
  __shared__ int64_t s_row[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int D = a.head_dim, Dv = a.v_dim, G = a.num_kv_heads;
  const int g = h / (a.num_heads / G);
  const int s = seq_of_row(a.query_start_loc, a.num_seqs, t);
  const int pos = a.seq_lens[s] - (a.query_start_loc[s + 1] - t);
  if (pos < 0) return;
  const int first = a.window_left >= 0 ? max(0, pos - a.window_left) : 0;
  const elem* q = static_cast<const elem*>(a.q) + static_cast<int64_t>(t) * a.q_stride_t + static_cast<int64_t>(h) * D;
  for (int d = lane; d < D; d += 64) s_q[d] = A::ld(q + d);
  const int32_t* bt = a.block_tables + static_cast<int64_t>(s) * a.block_table_stride;
  const elem* cache = static_cast<const elem*>(a.kv_cache);
  const int64_t row_elems = static_cast<int64_t>(G) * (D + Dv);
  const float ba = a.bias_mode ? a.bias_a[h] : 0.f, bb = a.bias_mode ? a.bias_b[h] : 0.f;
  float m = a.sink ? 0.f : -INFINITY, l = a.sink ? 1.f : 0.f;
  float acc[kMaxVChunks] = {0.f, 0.f, 0.f, 0.f};
  const int nvc = (Dv + 63) / 64;
  __syncthreads();
  for (int j0 = first; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float sc = -INFINITY;
    int64_t roff = 0;
    if (valid) {
      const int64_t blk = bt[j / a.block_size];
      roff = (blk * a.block_size + j % a.block_size) * row_elems + static_cast<int64_t>(g) * (D + Dv);
      const elem* k = cache + roff;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(s_q[d], A::ld(k + d), dot);
      sc = dot * a.scale - distance_bias(a.bias_mode, ba, bb, pos - j);
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float p = valid ? expf(sc - m_new) : 0.f;
    const float corr = expf(m - m_new);            // m = -inf only without a sink before the first tile: corr = 0, l = 0
    l = l * corr + wave_sum(p);
    m = m_new;
    __syncthreads();
    s_p[lane] = p;
    s_row[lane] = roff + D;
    __syncthreads();
    const int n = min(64, pos - j0 + 1);
#pragma unroll
    for (int cc = 0; cc < kMaxVChunks; ++cc) {
      if (cc < nvc) {
        const int c = cc * 64 + lane;
        float r = acc[cc] * corr;
        if (c < Dv)
          for (int jj = 0; jj < n; ++jj) r = fmaf(s_p[jj], A::ld(cache + s_row[jj] + c), r);
        acc[cc] = r;
      }
    }
  }
  elem* out = static_cast<elem*>(a.out) + (static_cast<int64_t>(t) * a.num_heads + h) * Dv;
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int cc = 0; cc < kMaxVChunks; ++cc) {
    const int c = cc * 64 + lane;
    if (cc < nvc && c < Dv) A::st(out + c, acc[cc] * inv);
  }
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_qk_norm_cache(const hymeta_qk_norm_cache_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_qk_norm_cache_args& a = *args;
  if (a.num_tokens < 0 || a.num_heads <= 0 || a.num_kv_heads <= 0 || a.head_dim <= 0 || a.v_dim <= 0 || a.block_size <= 0 ||
      a.num_blocks < 0)
    return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.qkv || (a.slot_mapping && !a.kv_cache)) return HYMETA_ERR_INVALID_ARG;
  if (a.qkv_stride_t < static_cast<int64_t>(a.num_heads + a.num_kv_heads) * a.head_dim + static_cast<int64_t>(a.num_kv_heads) * a.v_dim)
    return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(qk_norm_cache_kernel<ActBf16>, dim3(a.num_tokens), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(qk_norm_cache_kernel<ActF32>, dim3(a.num_tokens), dim3(256), 0, st, a);
  return launch_status();
}

extern "C" size_t hymeta_sink_attention_workspace_bytes(int32_t num_tokens, int32_t num_heads, int32_t v_dim, int32_t max_seq_len) {
  (void)num_tokens, (void)num_heads, (void)v_dim, (void)max_seq_len;
  return 0;
}

extern "C" int hymeta_sink_attention(const hymeta_sink_attention_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_sink_attention_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.num_heads <= 0 || a.num_kv_heads <= 0 || a.head_dim <= 0 || a.v_dim <= 0 ||
      a.block_size <= 0 || a.num_blocks < 0)
    return HYMETA_ERR_INVALID_ARG;
  if (a.num_heads % a.num_kv_heads != 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.head_dim > kMaxHeadDim || a.v_dim > 64 * kMaxVChunks) return HYMETA_ERR_UNSUPPORTED;
  if (a.bias_mode != HYMETA_BIAS_NONE && a.bias_mode != HYMETA_BIAS_LOG_DISTANCE) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.q || !a.kv_cache || !a.out || !a.block_tables || !a.query_start_loc || !a.seq_lens) return HYMETA_ERR_INVALID_ARG;
  if (a.bias_mode != HYMETA_BIAS_NONE && (!a.bias_a || !a.bias_b)) return HYMETA_ERR_INVALID_ARG;
  if (a.num_heads > 65535) return HYMETA_ERR_UNSUPPORTED;
  hipStream_t st = begin_launches(stream);
  const dim3 grid(a.num_tokens, a.num_heads);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(sink_attention_rows_kernel<ActBf16>, grid, dim3(64), 0, st, a);
  else hipLaunchKernelGGL(sink_attention_rows_kernel<ActF32>, grid, dim3(64), 0, st, a);
  return launch_status();
}
