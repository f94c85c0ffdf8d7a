// Router of a mixture of experts: fp32 logits from the rows and the router's matrix (and bias), the top_k largest
// (sigmoid scores normalised over the chosen and scaled, a softmax over the chosen logits alone, or a softmax over all
// outputs with a corrected, group-limited choice and identity experts); then the counting sort by expert that the grouped
// GEMMs of the routed block read.
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kSortThreads = 1024;

// grid = tokens in fours, 256 threads.  The experts' dot products over the workgroup, eight experts and four tokens a
// round (a weight is loaded once for the four tokens; the loads of a round are independent of each other; the partial
// sums meet through the waves and LDS in a fixed order); then wave w picks the top_k of token w: every lane scans the
// experts lane, lane + 64, ..., the wave reduces to the largest score and, among equals, the lowest expert.
constexpr int kRouteTokens = 4;

template <typename A>
__global__ __launch_bounds__(256) void moe_scores_topk_kernel(hymeta_moe_route_sigmoid_args a) {
  typedef typename A::elem elem;
  __shared__ float s_score[kRouteTokens][HYMETA_MOE_TABLE_MAX_EXPERTS];
  __shared__ float s_top[kRouteTokens][HYMETA_MOE_TABLE_MAX_EXPERTS];
  __shared__ float s_choice[kRouteTokens][HYMETA_MOE_TABLE_MAX_EXPERTS];      // (grouped choice) corrected, masked scores
  __shared__ float s_part[4][kRouteTokens][8];
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * kRouteTokens;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, E = a.num_experts;
  const bool softmax_chosen = a.score_mode == HYMETA_ROUTE_SOFTMAX_CHOSEN, grouped = a.score_mode == HYMETA_ROUTE_SOFTMAX_GROUPED;
  const int R = E + (grouped ? a.extra_rows : 0);          // rows of the router's matrix
  const int live = min(static_cast<int64_t>(kRouteTokens), a.num_tokens - t0);
  const elem* x[kRouteTokens];
#pragma unroll
  for (int i = 0; i < kRouteTokens; ++i) x[i] = static_cast<const elem*>(a.x) + (t0 + min(i, live - 1)) * a.x_stride_t;
  for (int e0 = 0; e0 < R; e0 += 8) {
    float acc[kRouteTokens][8] = {};
#pragma unroll 2
    for (int k = threadIdx.x; k < a.hidden; k += 256) {
      float xv[kRouteTokens], wv[8];
#pragma unroll
      for (int i = 0; i < kRouteTokens; ++i) xv[i] = A::ld(x[i] + k);
#pragma unroll
      for (int j = 0; j < 8; ++j) wv[j] = a.router_weight[static_cast<int64_t>(min(e0 + j, R - 1)) * a.hidden + k];
#pragma unroll
      for (int i = 0; i < kRouteTokens; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = fmaf(xv[i], wv[j], acc[i][j]);
    }
#pragma unroll
    for (int i = 0; i < kRouteTokens; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float v = wave_sum(acc[i][j]);
        if (lane == 0) s_part[wave][i][j] = v;
      }
    __syncthreads();
    if (threadIdx.x < kRouteTokens * 8) {
      const int i = threadIdx.x >> 3, j = threadIdx.x & 7;
      if (e0 + j < R) {
        const float z = (s_part[0][i][j] + s_part[1][i][j]) + (s_part[2][i][j] + s_part[3][i][j]) + ((a.router_bias && e0 + j < E) ? a.router_bias[e0 + j] : 0.f);
        s_score[i][e0 + j] = (softmax_chosen || grouped) ? z : sigmoid_exact(z);
      }
    }
    __syncthreads();
  }
  if (wave >= live) return;
  const int64_t t = t0 + wave;
  float* score = s_score[wave];
  if (grouped) {
    // the gate computed alongside, then softmax over all outputs (in place), the corrected scores, and the groups' mask
    if (a.extra_rows > 0 && lane == 0) a.extra_out[t] = sigmoid_exact(score[E]);
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, score[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) sum += expf(score[e] - mx);
    sum = wave_sum(sum);
    float* choice = s_choice[wave];
    for (int e = lane; e < E; e += 64) {
      const float p = expf(score[e] - mx) / sum;
      score[e] = p;
      choice[e] = p + (a.correction ? a.correction[e] : 0.f);
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
    const int NG = a.num_groups > 1 ? a.num_groups : 1, gsize = E / NG;
    if (NG > 1 && a.keep_groups < NG) {
      float* gbest = s_top[wave];
      for (int g = lane; g < NG; g += 64) {
        float b = -INFINITY;
        for (int e = g * gsize; e < (g + 1) * gsize; ++e) b = fmaxf(b, choice[e]);
        gbest[g] = b;
      }
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();
      for (int k = 0; k < a.keep_groups; ++k) {
        float best = -INFINITY;
        int arg = 0x7fffffff;
        for (int g = lane; g < NG; g += 64) {
          const float v = gbest[g];
          if (v != INFINITY && (v > best || arg == 0x7fffffff)) best = v, arg = g;      // INFINITY marks a kept group
        }
        const float top = wave_max(best);
        int cand = (best == top && arg != 0x7fffffff) ? arg : 0x7fffffff;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, 64));
        if (lane == 0 && cand != 0x7fffffff) gbest[cand] = INFINITY;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
      }
      for (int e = lane; e < E; e += 64)
        if (gbest[e / gsize] != INFINITY) choice[e] = -INFINITY;
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();
    }
    float identity = 0.f;
    for (int k = 0; k < a.top_k; ++k) {
      float best = -INFINITY;
      int arg = 0x7fffffff;
      for (int e = lane; e < E; e += 64) {
        const float v = choice[e];
        if (v > best) best = v, arg = e;
      }
      const float top = wave_max(best);
      int cand = best == top ? arg : 0x7fffffff;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, 64));
      if (cand == 0x7fffffff) cand = 0;             // (fewer candidates than top_k: refused on the host)
      const float wgt = score[cand] * a.scale;
      if (a.first_identity > 0 && cand >= a.first_identity) identity += wgt;
      if (lane == 0) {
        a.topk_ids[t * a.top_k + k] = cand;
        a.topk_weights[t * a.top_k + k] = wgt;
        choice[cand] = -INFINITY;                   // taken
      }
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();
    }
    if (a.first_identity > 0 && lane == 0) a.identity_weight[t] = identity;
    return;
  }
  float total = 0.f;
  for (int k = 0; k < a.top_k; ++k) {
    float best = -INFINITY;
    int arg = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = score[e];
      if (v > best) best = v, arg = e;            // ascending e: the first of equals stays
    }
    const float top = wave_max(best);
    int cand = best == top ? arg : 0x7fffffff;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, 64));
    total += top;
    if (lane == 0) {
      a.topk_ids[t * a.top_k + k] = cand;
      s_top[wave][k] = top;
      score[cand] = -INFINITY;                    // taken
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  if (softmax_chosen) {
    // the first chosen logit is the largest: exponentials of the differences to it, over their sum
    const float top0 = s_top[wave][0];
    float sum = 0.f;
    for (int k = 0; k < a.top_k; ++k) sum += expf(s_top[wave][k] - top0);
    for (int k = lane; k < a.top_k; k += 64) a.topk_weights[t * a.top_k + k] = expf(s_top[wave][k] - top0) / sum * a.scale;
    return;
  }
  const float inv = a.scale / (total + 1e-20f);
  for (int k = lane; k < a.top_k; k += 64) a.topk_weights[t * a.top_k + k] = s_top[wave][k] * inv;
}

// One workgroup: count the pairs per expert in LDS, prefix, scatter (the order inside an expert's run depends on the
// atomics' arrival; every pair's row is computed on its own, so the results do not).
__global__ __launch_bounds__(kSortThreads) void moe_sort_pairs_kernel(hymeta_moe_route_sigmoid_args a) {
  __shared__ int s_count[HYMETA_MOE_TABLE_MAX_EXPERTS];
  __shared__ int s_off[HYMETA_MOE_TABLE_MAX_EXPERTS + 1];
  // identity experts have no rows: their pairs are left out (pair_pos -1), and the offsets cover the experts before them
  const bool has_identity = a.score_mode == HYMETA_ROUTE_SOFTMAX_GROUPED && a.first_identity > 0;
  const int tid = threadIdx.x, E = has_identity ? a.first_identity : a.num_experts, P = a.num_tokens * a.top_k;
  for (int e = tid; e < E; e += kSortThreads) s_count[e] = 0;
  __syncthreads();
  for (int p = tid; p < P; p += kSortThreads)
    if (a.topk_ids[p] < E) atomicAdd(&s_count[a.topk_ids[p]], 1);
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
    if (e >= E) {
      a.pair_pos[p] = -1;
      continue;
    }
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
  if (a.score_mode != HYMETA_ROUTE_SIGMOID_SUM && a.score_mode != HYMETA_ROUTE_SOFTMAX_CHOSEN && a.score_mode != HYMETA_ROUTE_SOFTMAX_GROUPED)
    return HYMETA_ERR_UNSUPPORTED;
  if (a.score_mode == HYMETA_ROUTE_SOFTMAX_GROUPED) {
    const int ng = a.num_groups > 1 ? a.num_groups : 1;
    if (a.extra_rows < 0 || a.extra_rows > 1 || a.num_experts + a.extra_rows > HYMETA_MOE_TABLE_MAX_EXPERTS) return HYMETA_ERR_UNSUPPORTED;
    if (a.num_experts % ng != 0 || a.keep_groups < 1 || a.first_identity > a.num_experts) return HYMETA_ERR_INVALID_ARG;
    if (ng > 1 && a.keep_groups < ng && static_cast<int64_t>(a.keep_groups) * (a.num_experts / ng) < a.top_k) return HYMETA_ERR_INVALID_ARG;
    if (a.num_tokens > 0 && ((a.first_identity > 0 && !a.identity_weight) || (a.extra_rows > 0 && !a.extra_out))) return HYMETA_ERR_INVALID_ARG;
  }
  if (!a.expert_offsets) return HYMETA_ERR_INVALID_ARG;
  if (a.num_tokens > 0 && (!a.x || !a.router_weight || !a.topk_ids || !a.topk_weights || !a.sorted_pair || !a.pair_pos || a.x_stride_t < a.hidden))
    return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.num_tokens > 0) {
    if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(moe_scores_topk_kernel<ActBf16>, dim3((a.num_tokens + kRouteTokens - 1) / kRouteTokens), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(moe_scores_topk_kernel<ActF32>, dim3((a.num_tokens + kRouteTokens - 1) / kRouteTokens), dim3(256), 0, st, a);
  }
  hipLaunchKernelGGL(moe_sort_pairs_kernel, dim3(1), dim3(kSortThreads), 0, st, a);
  return launch_status();
}
