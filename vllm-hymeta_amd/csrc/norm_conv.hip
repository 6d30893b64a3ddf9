// fp32 residual stream: embedding rows, RMS norm (+ short causal convolution over time with a carried
// state) on the way into a sublayer, output norm + scaled residual add on the way out.
//
// The norm statistics and the convolution are fp32; the normed row is rounded to the activation type
// before the convolution reads it (it is what a norm kernel on its own would have stored, and what the
// carried state holds), so a row's value does not depend on whether its predecessors came from this
// step or from the state.
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kNormThreads = 256;
constexpr int kNormWaves = kNormThreads / 64;
constexpr int kMaxPerThread = 32;          // width <= 256 * 32 channels

template <typename A>
__global__ __launch_bounds__(kNormThreads) void embed_rows_kernel(hymeta_embed_rows_args a) {
  const int t = blockIdx.x;
  int64_t tok = a.token_ids[t];
  if (tok < 0 || tok >= a.vocab) tok = 0;          // ids are validated on the host; never read out of the table
  const typename A::elem* row = static_cast<const typename A::elem*>(a.table) + tok * a.width;
  float* out = a.out + static_cast<int64_t>(t) * a.width;
  for (int c = threadIdx.x; c < a.width; c += kNormThreads) out[c] = A::ld(row + c) + (a.add ? a.add[c] : 0.f);
}

// 1 / sqrt(mean(row^2) + eps) of an fp32 row, the same value in every thread.
__device__ __forceinline__ float inv_rms(const float* row, int width, float eps, float* red) {
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += kNormThreads) {
    const float v = row[c];
    ss += v * v;
  }
  ss = block_sum<kNormWaves>(ss, red);
  return 1.f / sqrtf(ss / static_cast<float>(width) + eps);
}

// One workgroup per token row.  Rows 1 .. taps - 2 of a portion are computed by the workgroup of its row 0, which is
// also the only one that touches the sequence's convolution state: it reads the old rows for the portion's first
// outputs and then writes the new ones.  A thread owns its channels in all of this, so no other thread waits for its
// reads or sees its writes.
template <typename A>
__global__ __launch_bounds__(kNormThreads) void norm_conv_kernel(hymeta_norm_conv_args a) {
  typedef typename A::elem elem;
  __shared__ float red[kNormWaves];
  const int t = blockIdx.x;
  const int taps = a.conv_weight ? a.taps : 1;
  const int hist = taps - 1;
  int s = 0, i = 0, q = 1, ctx = 0, slot = -1;
  int64_t row0 = t;
  if (hist > 0) {
    s = seq_of_row(a.query_start_loc, a.num_seqs, t);
    row0 = a.query_start_loc[s];
    i = t - static_cast<int>(row0);
    q = a.query_start_loc[s + 1] - static_cast<int>(row0);
    ctx = a.context_lens[s];
    slot = a.slot_idx ? a.slot_idx[s] : -1;
    if (i > 0 && i < hist) return;                     // computed by the portion's first workgroup
  }
  elem* state = (hist > 0 && a.conv_state && slot >= 0)
                    ? static_cast<elem*>(a.conv_state) + static_cast<int64_t>(slot) * hist * a.width : nullptr;
  const bool carried = state != nullptr && ctx > 0;
  const int todo = (hist > 0 && i == 0) ? min(hist, q) : 1;

  for (int ii = i; ii < i + todo; ++ii) {
    // the normed rows ii - hist .. ii of the portion (those at or after its start)
    float inv[HYMETA_CONV_MAX_TAPS];
    for (int j = 0; j < taps; ++j) {
      const int k = ii - hist + j;
      inv[j] = 0.f;
      if (k >= 0) inv[j] = inv_rms(a.x + (row0 + k) * a.x_stride_t, a.width, a.eps, red);
    }
    elem* out = static_cast<elem*>(a.out) + (row0 + ii) * static_cast<int64_t>(a.width);
    for (int c = threadIdx.x; c < a.width; c += kNormThreads) {
      const float w = a.weight_offset + a.weight[c];
      const float n = A::round(a.x[(row0 + ii) * a.x_stride_t + c] * inv[hist] * w);
      float acc = n;
      if (a.conv_weight != nullptr) {
        const float* cw = a.conv_weight + static_cast<int64_t>(c) * taps;
        acc = fmaf(cw[hist], n, acc);
        for (int j = 0; j < hist; ++j) {
          const int k = ii - hist + j;
          float v = 0.f;
          if (k >= 0) v = A::round(a.x[(row0 + k) * a.x_stride_t + c] * inv[j] * w);
          else if (carried) v = A::ld(state + static_cast<int64_t>(hist + k) * a.width + c);
          acc = fmaf(cw[j], v, acc);
        }
      }
      A::st(out + c, acc);
    }
  }

  if (hist > 0 && i == 0 && state != nullptr) {
    // new state row r = the normed row at portion index q - hist + r; indices before the portion come from the old
    // state (row q + r, which lies after the row being written: ascending r never reads a row already replaced)
    float inv[HYMETA_CONV_MAX_TAPS];
    for (int r = 0; r < hist; ++r) {
      const int k = q - hist + r;
      inv[r] = 0.f;
      if (k >= 0) inv[r] = inv_rms(a.x + (row0 + k) * a.x_stride_t, a.width, a.eps, red);
    }
    for (int c = threadIdx.x; c < a.width; c += kNormThreads) {
      const float w = a.weight_offset + a.weight[c];
      for (int r = 0; r < hist; ++r) {
        const int k = q - hist + r;
        float v = 0.f;
        if (k >= 0) v = A::round(a.x[(row0 + k) * a.x_stride_t + c] * inv[r] * w);
        else if (carried) v = A::ld(state + static_cast<int64_t>(hist + k) * a.width + c);
        A::st(state + static_cast<int64_t>(r) * a.width + c, v);
      }
    }
  }
}

template <typename A>
__global__ __launch_bounds__(kNormThreads) void norm_residual_kernel(hymeta_norm_residual_args a) {
  typedef typename A::elem elem;
  __shared__ float red[kNormWaves];
  const int64_t t = blockIdx.x;
  const elem* y = static_cast<const elem*>(a.y) + t * a.y_stride_t;
  float* x = a.x + t * a.x_stride_t;
  float v[kMaxPerThread];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < kMaxPerThread; ++u) {
    const int c = threadIdx.x + u * kNormThreads;
    v[u] = c < a.width ? A::ld(y + c) : 0.f;
    ss += v[u] * v[u];
  }
  ss = block_sum<kNormWaves>(ss, red);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(a.width) + a.eps);
#pragma unroll
  for (int u = 0; u < kMaxPerThread; ++u) {
    const int c = threadIdx.x + u * kNormThreads;
    if (c < a.width) {
      float r = x[c] + a.mult * (v[u] * inv * (a.weight_offset + a.weight[c]));
      if (a.post_add) r += a.post_add[c];
      x[c] = r;
    }
  }
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_embed_rows(const hymeta_embed_rows_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_embed_rows_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0 || a.vocab <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.token_ids || !a.table || !a.out) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(embed_rows_kernel<ActBf16>, dim3(a.num_tokens), dim3(kNormThreads), 0, st, a);
  else hipLaunchKernelGGL(embed_rows_kernel<ActF32>, dim3(a.num_tokens), dim3(kNormThreads), 0, st, a);
  return launch_status();
}

extern "C" int hymeta_norm_conv(const hymeta_norm_conv_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_norm_conv_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0 || a.num_seqs < 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.x || !a.weight || !a.out || a.x_stride_t < a.width) return HYMETA_ERR_INVALID_ARG;
  if (a.conv_weight) {
    if (a.taps < 1 || a.taps > HYMETA_CONV_MAX_TAPS) return HYMETA_ERR_UNSUPPORTED;
    if (a.taps > 1 && (a.num_seqs <= 0 || !a.query_start_loc || !a.context_lens)) return HYMETA_ERR_INVALID_ARG;
  }
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(norm_conv_kernel<ActBf16>, dim3(a.num_tokens), dim3(kNormThreads), 0, st, a);
  else hipLaunchKernelGGL(norm_conv_kernel<ActF32>, dim3(a.num_tokens), dim3(kNormThreads), 0, st, a);
  return launch_status();
}

extern "C" int hymeta_norm_residual(const hymeta_norm_residual_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_norm_residual_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.width > kNormThreads * kMaxPerThread) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.y || !a.weight || !a.x || a.x_stride_t < a.width || a.y_stride_t < a.width) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(norm_residual_kernel<ActBf16>, dim3(a.num_tokens), dim3(kNormThreads), 0, st, a);
  else hipLaunchKernelGGL(norm_residual_kernel<ActF32>, dim3(a.num_tokens), dim3(kNormThreads), 0, st, a);
  return launch_status();
}
