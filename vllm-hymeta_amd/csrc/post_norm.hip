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
  // four columns a round: their loads are in flight together (a short row is one round trip to memory, not four)
  for (int c0 = threadIdx.x; c0 < a.width; c0 += 4 * 256) {
    float h[4], hp[4], mx[4], lt[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = c0 + 256 * u;
      const bool ok = c < a.width;
      h[u] = ok ? x[c] : 0.f;
      hp[u] = ok ? (first ? (from_state ? st[c] : 0.f) : prev[c]) : 0.f;
      mx[u] = ok ? a.mix[c] : 0.f;
      lt[u] = (ok && first && st != nullptr) ? last[c] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = c0 + 256 * u;
      if (c >= a.width) continue;
      A::st(out + c, h[u] + (hp[u] - h[u]) * mx[u]);
      if (first && st != nullptr) st[c] = lt[u];
    }
  }
}

__device__ __forceinline__ float summed(const hymeta_add_group_norm_args& a, const float* x, const void* y, const void* y2, int c,
                                        bool bf) {
  float z = a.alpha * x[c];
  if (y) z += bf ? bf2f(static_cast<const uint16_t*>(y)[c]) : static_cast<const float*>(y)[c];
  if (y2) z += bf ? bf2f(static_cast<const uint16_t*>(y2)[c]) : static_cast<const float*>(y2)[c];
  return z;
}

// grid = rows; the groups one after the other, each with a sum over the workgroup.  Rows of up to kNormCached columns
// are read once: a thread keeps its columns of the sum in registers between the statistics and the scaling.
constexpr int kNormPerThread = 16, kNormCached = 256 * kNormPerThread;

// Mode 0: any shape, two passes over the row.  Mode 1: rows of up to kNormCached columns, read once, a thread keeps its
// columns between the statistics and the scaling.  Mode 2: the same with four consecutive columns per load and store
// (groups, strides and pointers in whole fours).
template <typename A, int Mode>
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
  float z[Mode ? kNormPerThread : 1];
  // column of this thread's value u
  auto col = [&](int u) { return Mode == 2 ? 4 * (static_cast<int>(threadIdx.x) + 256 * (u >> 2)) + (u & 3) : static_cast<int>(threadIdx.x) + 256 * u; };
  if (Mode == 1) {
#pragma unroll
    for (int u = 0; u < kNormPerThread; ++u) z[u] = col(u) < a.width ? summed(a, x, y, y2, col(u), bf) : 0.f;
  }
  if (Mode == 2) {
#pragma unroll
    for (int u = 0; u < kNormPerThread; u += 4) {
      const int c = col(u);
      float xv[4] = {}, yv[4] = {}, y2v[4] = {};
      if (c < a.width) {
        ActF32::ld4(x + c, xv);
        if (y) A::ld4(y + c, yv);
        if (y2) A::ld4(y2 + c, y2v);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float s = a.alpha * xv[e];
        if (y) s += yv[e];
        if (y2) s += y2v[e];
        z[u + e] = s;
      }
    }
  }
  for (int g = 0; g < a.groups; ++g) {
    const int lo = g * part;
    float ss = 0.f;
    if (Mode) {
#pragma unroll
      for (int u = 0; u < kNormPerThread; ++u)
        if (col(u) >= lo && col(u) < lo + part) ss = fmaf(z[u], z[u], ss);
    } else {
      for (int c = lo + threadIdx.x; c < lo + part; c += 256) {
        const float v = summed(a, x, y, y2, c, bf);
        ss = fmaf(v, v, ss);
      }
    }
    ss = block_sum<4>(ss, red);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(part) + a.eps);
    if (Mode == 2) {
#pragma unroll
      for (int u = 0; u < kNormPerThread; u += 4) {
        const int c = col(u);
        if (c >= lo && c < lo + part) {
          float wv[4], v[4];
          ActF32::ld4(a.weight + c, wv);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = z[u + e] * inv * wv[e];
          if (out) A::st4(out + c, v);
          if (a.in_place) ActF32::st4(x + c, v);
        }
      }
    } else if (Mode == 1) {
#pragma unroll
      for (int u = 0; u < kNormPerThread; ++u) {
        const int c = col(u);
        if (c >= lo && c < lo + part) {
          const float v = z[u] * inv * a.weight[c];
          if (out) A::st(out + c, v);
          if (a.in_place) x[c] = v;
        }
      }
    } else {
      for (int c = lo + threadIdx.x; c < lo + part; c += 256) {
        const float v = summed(a, x, y, y2, c, bf) * inv * a.weight[c];
        if (out) A::st(out + c, v);
        if (a.in_place) x[c] = v;
      }
    }
  }
}

template <typename A>
void launch_add_group_norm(const hymeta_add_group_norm_args& a, hipStream_t st) {
  const int elem = A::kDtype == HYMETA_BF16 ? 2 : 4;
  auto whole4 = [&](const void* p, int64_t stride, int bytes) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) % (4 * bytes) == 0 && stride % 4 == 0); };
  const bool fours = (a.width / a.groups) % 4 == 0 && whole4(a.x, a.x_stride_t, 4) && whole4(a.y, a.y_stride_t, elem) &&
                     whole4(a.y2, a.y2_stride_t, elem) && whole4(a.out, 0, elem) && whole4(a.weight, 0, 4);
  const dim3 grid(a.num_tokens), block(256);
  if (a.width > kNormCached) hipLaunchKernelGGL((add_group_norm_kernel<A, 0>), grid, block, 0, st, a);
  else if (fours) hipLaunchKernelGGL((add_group_norm_kernel<A, 2>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((add_group_norm_kernel<A, 1>), grid, block, 0, st, a);
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
  if (a.act_dtype == HYMETA_BF16) launch_add_group_norm<ActBf16>(a, st);
  else launch_add_group_norm<ActF32>(a, st);
  return launch_status();
}
