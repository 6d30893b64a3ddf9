// minGRU recurrence over a step's rows: per channel S <- (1 - z) S + z cand, out = S * silu(g), with the state
// fp32 in registers and carried between steps in a slot-indexed tensor.
//
// The recurrence is linear in S (S' = a S + b with a = 1 - z, b = z cand), so a portion of a prompt is scanned in
// parallel: a workgroup owns 64 channels of one sequence, its waves take consecutive runs of kRun rows, reduce each
// run to its (product of a, value from zero), pass the carry over the waves through LDS and then replay their run
// from the right starting state.  Sequences with one row (decode) run the one-wave form, which is the plain update;
// steps with portions of thousands of rows cut them into segments (below).
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kRun = 8;              // rows per wave and round
constexpr int kScanWaves = 8;        // waves of the prompt form

// Long portions are cut into segments of kSegment rows that run in workgroups of their own, in three launches:
// kSummarize scans every segment from a zero state and keeps (product of a, end value); a small kernel chains these over
// a sequence's segments into every segment's starting state (and the sequence's final state); kApply scans again from
// the right starting states and writes the outputs.
enum : int { kWhole = 0, kSummarize = 1, kApply = 2 };
constexpr int kSegment = 512;

// workspace: [3][num_seqs][segments][width] floats: products, end values, starting states
__device__ __forceinline__ float* seg_ptr(const hymeta_mingru_args& a, int what, int s, int seg, int segments) {
  return static_cast<float*>(a.workspace) + ((static_cast<size_t>(what) * a.num_seqs + s) * segments + seg) * a.width;
}

template <typename A, int Waves, int Mode>
__global__ __launch_bounds__(64 * Waves) void mingru_kernel(hymeta_mingru_args a, int segments) {
  typedef typename A::elem elem;
  __shared__ float s_a[Waves][64], s_b[Waves][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int s = blockIdx.y, seg = blockIdx.z;
  const int c = blockIdx.x * 64 + lane;
  const bool live = c < a.width;
  int64_t row0 = a.query_start_loc[s];
  int q = a.query_start_loc[s + 1] - static_cast<int>(row0);
  if (Mode != kWhole) {              // this workgroup's segment of the portion
    if (seg * kSegment >= q) return;
    row0 += seg * kSegment;
    q = min(kSegment, q - seg * kSegment);
  }
  if (q <= 0) return;
  const int slot = a.slot_idx[s];
  const int W = a.width;
  float carry = 0.f, prod = 1.f;
  if (Mode == kWhole && live && slot >= 0 && a.context_lens[s] > 0) carry = a.state[static_cast<int64_t>(slot) * W + c];
  if (Mode == kApply && live) carry = seg_ptr(a, 2, s, seg, segments)[c];
  const elem* zug = static_cast<const elem*>(a.zug);
  elem* out = static_cast<elem*>(a.out);

  // the raw projections of a round are loaded one round ahead of their use
  float rz[kRun], ru[kRun], rg[kRun];
  auto load = [&](int base, float (&z)[kRun], float (&u)[kRun], float (&g)[kRun]) {
    const int lo = base + wave * kRun;
#pragma unroll
    for (int l = 0; l < kRun; ++l) {
      z[l] = u[l] = g[l] = 0.f;
      if (live && lo + l < q) {
        const elem* r = zug + (row0 + lo + l) * a.zug_stride_t;
        z[l] = A::ld(r + c), u[l] = A::ld(r + W + c), g[l] = A::ld(r + 2 * W + c);
      }
    }
  };
  load(0, rz, ru, rg);
  for (int base = 0; base < q; base += kRun * Waves) {
    const int lo = base + wave * kRun;
    float nz[kRun], nu[kRun], ng[kRun];
    if (base + kRun * Waves < q) load(base + kRun * Waves, nz, nu, ng);
    float av[kRun], bv[kRun], gv[kRun];
#pragma unroll
    for (int l = 0; l < kRun; ++l) {
      av[l] = 1.f, bv[l] = 0.f, gv[l] = 0.f;
      if (live && lo + l < q) {
        const float z = A::sigmoid(rz[l]);
        const float cand = ru[l] >= 0.f ? ru[l] + 0.5f : A::sigmoid(ru[l]);
        av[l] = 1.f - z;
        bv[l] = z * cand;
        gv[l] = rg[l] * A::sigmoid(rg[l]);
      }
    }
    float S = carry;
    if (Waves > 1) {
      float pa = 1.f, pb = 0.f;
#pragma unroll
      for (int l = 0; l < kRun; ++l) {
        pb = fmaf(av[l], pb, bv[l]);
        pa *= av[l];
      }
      __syncthreads();                 // the round before has read the arrays
      s_a[wave][lane] = pa;
      s_b[wave][lane] = pb;
      __syncthreads();
      float next = carry;
#pragma unroll
      for (int w = 0; w < Waves; ++w) {
        if (w == wave) S = next;
        next = fmaf(s_a[w][lane], next, s_b[w][lane]);
        if (Mode == kSummarize) prod *= s_a[w][lane];
      }
      carry = next;
    }
#pragma unroll
    for (int l = 0; l < kRun; ++l) {
      S = fmaf(av[l], S, bv[l]);
      if (Mode != kSummarize && live && lo + l < q) A::st(out + (row0 + lo + l) * W + c, S * gv[l]);
    }
    if (Waves == 1) carry = S;
#pragma unroll
    for (int l = 0; l < kRun; ++l) rz[l] = nz[l], ru[l] = nu[l], rg[l] = ng[l];
  }
  if (Mode == kWhole && live && slot >= 0 && wave == 0) a.state[static_cast<int64_t>(slot) * W + c] = carry;
  if (Mode == kSummarize && live && wave == 0) {
    seg_ptr(a, 0, s, seg, segments)[c] = prod;
    seg_ptr(a, 1, s, seg, segments)[c] = carry;
  }
}

// grid = (channel tiles, sequences): a thread chains its channel over the sequence's segments.
__global__ __launch_bounds__(64) void mingru_chain_kernel(hymeta_mingru_args a, int segments) {
  const int s = blockIdx.y, c = blockIdx.x * 64 + threadIdx.x;
  if (c >= a.width) return;
  const int q = a.query_start_loc[s + 1] - a.query_start_loc[s];
  if (q <= 0) return;
  const int slot = a.slot_idx[s];
  float S = 0.f;
  if (slot >= 0 && a.context_lens[s] > 0) S = a.state[static_cast<int64_t>(slot) * a.width + c];
  const int n = (q + kSegment - 1) / kSegment;
  for (int seg = 0; seg < n; ++seg) {
    seg_ptr(a, 2, s, seg, segments)[c] = S;
    S = fmaf(seg_ptr(a, 0, s, seg, segments)[c], S, seg_ptr(a, 1, s, seg, segments)[c]);
  }
  if (slot >= 0) a.state[static_cast<int64_t>(slot) * a.width + c] = S;
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" size_t hymeta_mingru_workspace_bytes(int32_t num_seqs, int32_t width, int32_t max_query_len) {
  if (num_seqs <= 0 || width <= 0 || max_query_len < 4 * kSegment) return 0;
  const size_t segments = (static_cast<size_t>(max_query_len) + kSegment - 1) / kSegment;
  return 3 * static_cast<size_t>(num_seqs) * segments * width * sizeof(float);
}

template <typename A>
static int launch_mingru(const hymeta_mingru_args& a, hipStream_t st) {
  const dim3 tiles((a.width + 63) / 64, a.num_seqs);
  const size_t need = hymeta_mingru_workspace_bytes(a.num_seqs, a.width, a.max_query_len);
  if (need > 0) {
    if (!a.workspace || a.workspace_bytes < need) return HYMETA_ERR_WORKSPACE;
    const int segments = (a.max_query_len + kSegment - 1) / kSegment;
    const dim3 grid(tiles.x, tiles.y, segments);
    hipLaunchKernelGGL((mingru_kernel<A, kScanWaves, kSummarize>), grid, dim3(64 * kScanWaves), 0, st, a, segments);
    hipLaunchKernelGGL(mingru_chain_kernel, tiles, dim3(64), 0, st, a, segments);
    hipLaunchKernelGGL((mingru_kernel<A, kScanWaves, kApply>), grid, dim3(64 * kScanWaves), 0, st, a, segments);
  } else if (a.max_query_len > kRun) {
    hipLaunchKernelGGL((mingru_kernel<A, kScanWaves, kWhole>), tiles, dim3(64 * kScanWaves), 0, st, a, 1);
  } else {
    hipLaunchKernelGGL((mingru_kernel<A, 1, kWhole>), tiles, dim3(64), 0, st, a, 1);
  }
  return launch_status();
}

extern "C" int hymeta_mingru(const hymeta_mingru_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_mingru_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.width <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.zug || !a.state || !a.out || !a.query_start_loc || !a.context_lens || !a.slot_idx) return HYMETA_ERR_INVALID_ARG;
  if (a.zug_stride_t < 3 * static_cast<int64_t>(a.width)) return HYMETA_ERR_INVALID_ARG;
  if (a.num_seqs > 65535) return HYMETA_ERR_UNSUPPORTED;
  hipStream_t st = begin_launches(stream);
  return a.act_dtype == HYMETA_BF16 ? launch_mingru<ActBf16>(a, st) : launch_mingru<ActF32>(a, st);
}
