// Elementwise activations between two projections: the clamped gated unit of the experts, xIELU of the dense
// feed-forward, and an output gate.  act_dtype in and out, fp32 inside.
#include "act_types.h"

namespace hymeta {

namespace {

__device__ __forceinline__ float clamped_glu(float gate, float up, float limit, float alpha) {
  const float g = fminf(gate, limit);
  const float u = fminf(fmaxf(up, -limit), limit);
  return g * sigmoid_exact(alpha * g) * (u + 1.f);
}

__device__ __forceinline__ float xielu(float z, float a_pos, float a_neg) {
  return z > 0.f ? fmaf(a_pos * z, z, 0.5f * z) : fmaf(a_neg, expm1f(z) - z, 0.5f * z);
}

template <typename A>
__global__ __launch_bounds__(256) void activation_kernel(hymeta_activation_args a) {
  typedef typename A::elem elem;
  const int rows = a.num_rows_dev ? min(*a.num_rows_dev, a.num_rows) : a.num_rows;
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const elem* x = static_cast<const elem*>(a.x) + r * a.x_stride;
    elem* out = static_cast<elem*>(a.out) + r * a.out_stride;
    // four columns a round, their loads in flight together
    const elem* g = a.gate ? static_cast<const elem*>(a.gate) + r * a.gate_stride : nullptr;
    for (int c0 = threadIdx.x; c0 < a.n; c0 += 4 * 256) {
      float v0[4], v1[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + 256 * u;
        const bool ok = c < a.n;
        v0[u] = ok ? A::ld(x + c) : 0.f;
        v1[u] = !ok ? 0.f : a.kind == HYMETA_ACT_CLAMPED_GLU ? A::ld(x + a.n + c) : a.kind == HYMETA_ACT_SIGMOID_MUL ? A::ld(g + c) : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + 256 * u;
        if (c >= a.n) continue;
        float v;
        if (a.kind == HYMETA_ACT_CLAMPED_GLU) v = clamped_glu(v0[u], v1[u], a.p0, a.p1);
        else if (a.kind == HYMETA_ACT_XIELU) v = xielu(v0[u], a.p0, a.p1);
        else v = v0[u] * sigmoid_exact(v1[u]);
        A::st(out + c, v);
      }
    }
  }
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_activation(const hymeta_activation_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_activation_args& a = *args;
  if (a.num_rows < 0 || a.n <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.kind != HYMETA_ACT_CLAMPED_GLU && a.kind != HYMETA_ACT_XIELU && a.kind != HYMETA_ACT_SIGMOID_MUL) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_rows == 0) return HYMETA_OK;
  if (!a.x || !a.out || (a.kind == HYMETA_ACT_SIGMOID_MUL && !a.gate)) return HYMETA_ERR_INVALID_ARG;
  const int64_t in_cols = a.kind == HYMETA_ACT_CLAMPED_GLU ? 2 * static_cast<int64_t>(a.n) : a.n;
  if (a.x_stride < in_cols || a.out_stride < a.n || (a.kind == HYMETA_ACT_SIGMOID_MUL && a.gate_stride < a.n)) return HYMETA_ERR_INVALID_ARG;
  const int grid = a.num_rows < 65535 ? a.num_rows : 65535;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(activation_kernel<ActBf16>, dim3(grid), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(activation_kernel<ActF32>, dim3(grid), dim3(256), 0, st, a);
  return launch_status();
}
