// Post-norm decoder blocks on an fp32 stream: the token shift in front of a mixer and the grouped RMS norm
// after the sum of the scaled stream and a sublayer's output.
#include "act_types.h"

namespace hymeta {

namespace {

// grid = rows.  The first row of a portion reads the sequence's state and then, element by element in the same
// thread, replaces it with the portion's last row: no other workgroup touches that state.
template <typename A>
__global__ __launch_bounds__(256) void token_shift_kernel(hymeta_token_shift_args a) {
  typedef typename A::elem elem;
  const int t = blockIdx.x;
  const int s = seq_of_row(a.query_start_loc, a.num_seqs, t);
  const int r0 = a.query_start_loc[s], r1 = a.query_start_loc[s + 1];
  const int slot = a.slot_idx ? a.slot_idx[s] : -1;
  const float* x = a.x + static_cast<int64_t>(t) * a.x_stride_t;
  elem* out = static_cast<elem*>(a.out) + static_cast<int64_t>(t) * a.width;
  const bool first = t == r0;
  const bool from_state = first && slot >= 0 && a.state != nullptr && a.context_lens[s] > 0;
  const float* prev = first ? nullptr : x - a.x_stride_t;
  float* st = (slot >= 0 && a.state != nullptr) ? a.state + static_cast<int64_t>(slot) * a.width : nullptr;
  const float* last = a.x + static_cast<int64_t>(r1 - 1) * a.x_stride_t;
  for (int c = threadIdx.x; c < a.width; c += 256) {
    const float h = x[c];
    const float hp = first ? (from_state ? st[c] : 0.f) : prev[c];
    A::st(out + c, h + (hp - h) * a.mix[c]);
    if (first && st != nullptr) st[c] = last[c];
  }
}

__device__ __forceinline__ float summed(const hymeta_add_group_norm_args& a, const float* x, const void* y, const void* y2, int c,
                                        bool bf) {
  float z = a.alpha * x[c];
  if (y) z += bf ? bf2f(static_cast<const uint16_t*>(y)[c]) : static_cast<const float*>(y)[c];
  if (y2) z += bf ? bf2f(static_cast<const uint16_t*>(y2)[c]) : static_cast<const float*>(y2)[c];
  return z;
}

// grid = rows; the groups one after the other, each with a sum over the workgroup.
template <typename A>
__global__ __launch_bounds__(256) void add_group_norm_kernel(hymeta_add_group_norm_args a) {
  typedef typename A::elem elem;
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  constexpr bool bf = A::kDtype == HYMETA_BF16;
  float* x = a.x + t * a.x_stride_t;
  const elem* y = a.y ? static_cast<const elem*>(a.y) + t * a.y_stride_t : nullptr;
  const elem* y2 = a.y2 ? static_cast<const elem*>(a.y2) + t * a.y2_stride_t : nullptr;
  elem* out = a.out ? static_cast<elem*>(a.out) + t * a.width : nullptr;
  const int part = a.width / a.groups;
  for (int g = 0; g < a.groups; ++g) {
    const int lo = g * part;
    float ss = 0.f;
    for (int c = lo + threadIdx.x; c < lo + part; c += 256) {
      const float z = summed(a, x, y, y2, c, bf);
      ss = fmaf(z, z, ss);
    }
    ss = block_sum<4>(ss, red);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(part) + a.eps);
    for (int c = lo + threadIdx.x; c < lo + part; c += 256) {
      const float v = summed(a, x, y, y2, c, bf) * inv * a.weight[c];
      if (out) A::st(out + c, v);
      if (a.in_place) x[c] = v;
    }
  }
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_token_shift(const hymeta_token_shift_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_token_shift_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.width <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.x || !a.mix || !a.out || !a.query_start_loc || !a.context_lens || a.x_stride_t < a.width) return HYMETA_ERR_INVALID_ARG;
  if (a.state && !a.slot_idx) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(token_shift_kernel<ActBf16>, dim3(a.num_tokens), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(token_shift_kernel<ActF32>, dim3(a.num_tokens), dim3(256), 0, st, a);
  return launch_status();
}

extern "C" int hymeta_add_group_norm(const hymeta_add_group_norm_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_add_group_norm_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0 || a.groups <= 0 || a.width % a.groups != 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.x || !a.weight || a.x_stride_t < a.width || (!a.out && !a.in_place)) return HYMETA_ERR_INVALID_ARG;
  if ((a.y && a.y_stride_t < a.width) || (a.y2 && a.y2_stride_t < a.width)) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(add_group_norm_kernel<ActBf16>, dim3(a.num_tokens), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(add_group_norm_kernel<ActF32>, dim3(a.num_tokens), dim3(256), 0, st, a);
  return launch_status();
}
