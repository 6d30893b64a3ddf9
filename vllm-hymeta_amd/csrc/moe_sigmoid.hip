// Router of a mixture of experts with sigmoid scores: fp32 logits from the rows and the router's matrix, the top_k
// largest scores, weights normalised over the chosen and scaled; then the counting sort by expert that the grouped
// GEMMs of the routed block read.
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kSortThreads = 1024;

// grid = tokens, 256 threads.  A wave per expert's dot product (lanes over the hidden size, a fixed order of
// summation); then wave 0 picks the top_k: every lane scans the experts lane, lane + 64, ..., the wave reduces to the
// largest score and, among equals, the lowest expert.
template <typename A>
__global__ __launch_bounds__(256) void moe_scores_topk_kernel(hymeta_moe_route_sigmoid_args a) {
  typedef typename A::elem elem;
  __shared__ float s_score[HYMETA_MOE_TABLE_MAX_EXPERTS];
  __shared__ float s_top[HYMETA_MOE_TABLE_MAX_EXPERTS];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, E = a.num_experts;
  const elem* x = static_cast<const elem*>(a.x) + t * a.x_stride_t;
  for (int e = wave; e < E; e += 4) {
    const float* w = a.router_weight + static_cast<int64_t>(e) * a.hidden;
    float z = 0.f;
    for (int k = lane; k < a.hidden; k += 64) z = fmaf(A::ld(x + k), w[k], z);
    z = wave_sum(z);
    if (lane == 0) s_score[e] = sigmoid_exact(z);
  }
  __syncthreads();
  if (wave != 0) return;
  float total = 0.f;
  for (int k = 0; k < a.top_k; ++k) {
    float best = -2.f;
    int arg = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = s_score[e];
      if (v > best) best = v, arg = e;            // ascending e: the first of equals stays
    }
    const float top = wave_max(best);
    int cand = best == top ? arg : 0x7fffffff;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, 64));
    total += top;
    if (lane == 0) {
      a.topk_ids[t * a.top_k + k] = cand;
      s_top[k] = top;
      s_score[cand] = -1.f;                       // scores are >= 0: taken
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  const float inv = a.scale / (total + 1e-20f);
  for (int k = lane; k < a.top_k; k += 64) a.topk_weights[t * a.top_k + k] = s_top[k] * inv;
}

// One workgroup: count the pairs per expert in LDS, prefix, scatter (the order inside an expert's run depends on the
// atomics' arrival; every pair's row is computed on its own, so the results do not).
__global__ __launch_bounds__(kSortThreads) void moe_sort_pairs_kernel(hymeta_moe_route_sigmoid_args a) {
  __shared__ int s_count[HYMETA_MOE_TABLE_MAX_EXPERTS];
  __shared__ int s_off[HYMETA_MOE_TABLE_MAX_EXPERTS + 1];
  const int tid = threadIdx.x, E = a.num_experts, P = a.num_tokens * a.top_k;
  for (int e = tid; e < E; e += kSortThreads) s_count[e] = 0;
  __syncthreads();
  for (int p = tid; p < P; p += kSortThreads) atomicAdd(&s_count[a.topk_ids[p]], 1);
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      s_off[e] = run;
      run += s_count[e];
    }
    s_off[E] = run;
  }
  __syncthreads();
  for (int e = tid; e <= E; e += kSortThreads) a.expert_offsets[e] = s_off[e];
  for (int e = tid; e < E; e += kSortThreads) s_count[e] = 0;
  __syncthreads();
  for (int p = tid; p < P; p += kSortThreads) {
    const int e = a.topk_ids[p];
    const int pos = s_off[e] + atomicAdd(&s_count[e], 1);
    a.sorted_pair[pos] = p;
    a.pair_pos[p] = pos;
  }
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_moe_route_sigmoid(const hymeta_moe_route_sigmoid_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_moe_route_sigmoid_args& a = *args;
  if (a.num_tokens < 0 || a.num_experts <= 0 || a.top_k <= 0 || a.hidden <= 0) return HYMETA_ERR_INVALID_ARG;
  if (a.num_experts > HYMETA_MOE_TABLE_MAX_EXPERTS || a.top_k > a.num_experts) return HYMETA_ERR_UNSUPPORTED;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (!a.expert_offsets) return HYMETA_ERR_INVALID_ARG;
  if (a.num_tokens > 0 && (!a.x || !a.router_weight || !a.topk_ids || !a.topk_weights || !a.sorted_pair || !a.pair_pos || a.x_stride_t < a.hidden))
    return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.num_tokens > 0) {
    if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(moe_scores_topk_kernel<ActBf16>, dim3(a.num_tokens), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(moe_scores_topk_kernel<ActF32>, dim3(a.num_tokens), dim3(256), 0, st, a);
  }
  hipLaunchKernelGGL(moe_sort_pairs_kernel, dim3(1), dim3(kSortThreads), 0, st, a);
  return launch_status();
}
