// Mixture of experts chosen by a table lookup on the token id, and the shape- and type-generic forms of the routed
// block's grouped GEMM and combine (fp32 or bf16 operands, any K and N) that run where the MFMA tiles of moe.hip do
// not take the problem.
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kRouteThreads = 1024;

// One workgroup: count the pairs per expert in LDS, prefix, scatter.  The order of the pairs inside an expert's run
// depends on the atomics' arrival; every pair's row is computed on its own, so the results do not.
__global__ __launch_bounds__(kRouteThreads) void moe_route_table_kernel(hymeta_moe_route_table_args a) {
  __shared__ int s_count[HYMETA_MOE_TABLE_MAX_EXPERTS];
  __shared__ int s_off[HYMETA_MOE_TABLE_MAX_EXPERTS + 1];
  const int tid = threadIdx.x, E = a.num_experts, P = a.num_tokens * a.top_k;
  for (int e = tid; e < E; e += kRouteThreads) s_count[e] = 0;
  __syncthreads();
  const float w = 1.f / static_cast<float>(a.top_k);
  for (int p = tid; p < P; p += kRouteThreads) {
    int64_t tok = a.token_ids[p / a.top_k];
    if (tok < 0 || tok >= a.vocab) tok = 0;
    int e = a.table[tok * a.top_k + p % a.top_k];
    if (e < 0 || e >= E) e = 0;
    a.topk_ids[p] = e;
    a.topk_weights[p] = w;
    atomicAdd(&s_count[e], 1);
  }
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
  for (int e = tid; e <= E; e += kRouteThreads) a.expert_offsets[e] = s_off[e];
  for (int e = tid; e < E; e += kRouteThreads) s_count[e] = 0;
  __syncthreads();
  for (int p = tid; p < P; p += kRouteThreads) {
    const int e = a.topk_ids[p];                 // this thread's own store above
    const int pos = s_off[e] + atomicAdd(&s_count[e], 1);
    a.sorted_pair[pos] = p;
    a.pair_pos[p] = pos;
  }
}

constexpr int kBM = 64, kBN = 64, kBK = 16;

// 64 x 64 output tile of one expert's rows, 4 x 4 outputs per thread, operands widened to fp32 in LDS.
template <typename A, bool Gated>
__global__ __launch_bounds__(256) void moe_gemm_any_kernel(hymeta_moe_gemm_any_args a) {
  typedef typename A::elem elem;
  __shared__ float s_x[kBK][kBM + 4];
  __shared__ float s_w[Gated ? 2 : 1][kBK][kBN + 4];
  const int tid = threadIdx.x;
  int e = -1, row_lo = 0, row_hi = 0;
  {
    int t = blockIdx.y;
    for (int i = 0; i < a.num_experts; ++i) {
      const int lo = a.expert_offsets[i], hi = a.expert_offsets[i + 1];
      const int tiles = (hi - lo + kBM - 1) / kBM;
      if (t < tiles) {
        e = i;
        row_lo = lo + t * kBM;
        row_hi = hi;
        break;
      }
      t -= tiles;
    }
  }
  if (e < 0) return;
  const int col0 = blockIdx.x * kBN;
  const int lr = tid >> 2, lk = (tid & 3) * 4;          // staging: row / column lr, k offsets lk .. lk + 3
  const int slot_l = row_lo + lr;
  const elem* xrow = nullptr;
  if (slot_l < row_hi) {
    const int src = a.a_rows ? a.a_rows[slot_l] / a.a_rows_div : slot_l;
    xrow = static_cast<const elem*>(a.x) + static_cast<int64_t>(src) * a.x_stride_m;
  }
  const elem* wbase = static_cast<const elem*>(a.weights) + static_cast<int64_t>(e) * a.w_stride_e;
  const int ncol = col0 + lr;
  const elem* wrow = ncol < a.N ? wbase + static_cast<int64_t>(ncol) * a.K : nullptr;
  const elem* wrow2 = (Gated && ncol < a.N) ? wbase + static_cast<int64_t>(a.N + ncol) * a.K : nullptr;

  const int ty = tid >> 4, tx = tid & 15;
  float acc[4][4] = {}, acc2[4][4] = {};
  for (int k0 = 0; k0 < a.K; k0 += kBK) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + lk + u;
      s_x[lk + u][lr] = (xrow && k < a.K) ? A::ld(xrow + k) : 0.f;
      s_w[0][lk + u][lr] = (wrow && k < a.K) ? A::ld(wrow + k) : 0.f;
      if (Gated) s_w[1][lk + u][lr] = (wrow2 && k < a.K) ? A::ld(wrow2 + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kBK; ++kk) {
      float xv[4], wv[4], wv2[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        xv[u] = s_x[kk][ty * 4 + u];
        wv[u] = s_w[0][kk][tx * 4 + u];
        if (Gated) wv2[u] = s_w[1][kk][tx * 4 + u];
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          acc[r][c] = fmaf(xv[r], wv[c], acc[r][c]);
          if (Gated) acc2[r][c] = fmaf(xv[r], wv2[c], acc2[r][c]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int slot = row_lo + ty * 4 + r;
    if (slot >= row_hi) continue;
    float sc = 1.f;
    if (a.row_scale) sc = a.row_scale[a.scale_rows ? a.scale_rows[slot] : slot];
    elem* orow = static_cast<elem*>(a.out) + static_cast<int64_t>(slot) * a.out_stride_m;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int n = col0 + tx * 4 + c;
      if (n >= a.N) continue;
      float v = acc[r][c];
      if (Gated) {
        const float gte = A::round(v), up = A::round(acc2[r][c]);   // the two projections' outputs as a GEMM would store them
        if (a.gated == HYMETA_GLU_CLAMPED) {
          const float gc = fminf(gte, a.act_limit), uc = fminf(fmaxf(up, -a.act_limit), a.act_limit);
          v = gc * sigmoid_exact(a.act_alpha * gc) * (uc + 1.f);
        } else {
          v = gte * sigmoid_exact(gte) * up;
        }
      }
      if (!Gated && a.gated == HYMETA_GLU_RELU2) {
        const float r = fmaxf(A::round(v), 0.f);       // the projection's output as a GEMM would store it
        v = r * r;
      }
      A::st(orow + n, v * sc);
    }
  }
}

template <typename A>
__global__ __launch_bounds__(256) void moe_combine_any_kernel(hymeta_moe_combine_any_args a) {
  typedef typename A::elem elem;
  const int64_t t = blockIdx.x;
  elem* out = static_cast<elem*>(a.out) + t * a.out_stride_m;
  for (int c = threadIdx.x; c < a.width; c += 256) {
    float s = 0.f;
    for (int k = 0; k < a.top_k; ++k) {
      const int pos = a.pair_pos[t * a.top_k + k];
      if (pos >= 0) s += A::ld(static_cast<const elem*>(a.y) + static_cast<int64_t>(pos) * a.y_stride_m + c);
    }
    A::st(out + c, s);
  }
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_moe_route_table(const hymeta_moe_route_table_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_moe_route_table_args& a = *args;
  if (a.num_tokens < 0 || a.num_experts <= 0 || a.top_k <= 0 || a.vocab <= 0) return HYMETA_ERR_INVALID_ARG;
  if (a.num_experts > HYMETA_MOE_TABLE_MAX_EXPERTS || a.top_k > a.num_experts) return HYMETA_ERR_UNSUPPORTED;
  if (!a.expert_offsets) return HYMETA_ERR_INVALID_ARG;
  if (a.num_tokens > 0 && (!a.token_ids || !a.table || !a.topk_ids || !a.topk_weights || !a.sorted_pair || !a.pair_pos))
    return HYMETA_ERR_INVALID_ARG;
  hipLaunchKernelGGL(moe_route_table_kernel, dim3(1), dim3(kRouteThreads), 0, begin_launches(stream), a);
  return launch_status();
}

extern "C" int hymeta_moe_gemm_any(const hymeta_moe_gemm_any_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_moe_gemm_any_args& a = *args;
  if (a.max_rows < 0 || a.K <= 0 || a.N <= 0 || a.num_experts <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.gated < HYMETA_GLU_NONE || a.gated > HYMETA_GLU_RELU2) return HYMETA_ERR_UNSUPPORTED;
  if (a.max_rows == 0) return HYMETA_OK;
  if (!a.x || !a.weights || !a.out || !a.expert_offsets) return HYMETA_ERR_INVALID_ARG;
  if (a.a_rows != nullptr && a.a_rows_div <= 0) return HYMETA_ERR_INVALID_ARG;
  if (a.x_stride_m < a.K || a.out_stride_m < a.N) return HYMETA_ERR_INVALID_ARG;
  const int64_t tiles = (static_cast<int64_t>(a.max_rows) + kBM - 1) / kBM + a.num_experts;
  if (tiles > 65535) return HYMETA_ERR_UNSUPPORTED;
  const dim3 grid((a.N + kBN - 1) / kBN, static_cast<unsigned>(tiles));
  hipStream_t st = begin_launches(stream);
  const bool bf = a.act_dtype == HYMETA_BF16;
  if (a.gated == HYMETA_GLU_SILU || a.gated == HYMETA_GLU_CLAMPED) {
    if (bf) hipLaunchKernelGGL((moe_gemm_any_kernel<ActBf16, true>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((moe_gemm_any_kernel<ActF32, true>), grid, dim3(256), 0, st, a);
  } else {
    if (bf) hipLaunchKernelGGL((moe_gemm_any_kernel<ActBf16, false>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((moe_gemm_any_kernel<ActF32, false>), grid, dim3(256), 0, st, a);
  }
  return launch_status();
}

extern "C" int hymeta_moe_combine_any(const hymeta_moe_combine_any_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_moe_combine_any_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0 || a.top_k <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.y || !a.out || !a.pair_pos) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(moe_combine_any_kernel<ActBf16>, dim3(a.num_tokens), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(moe_combine_any_kernel<ActF32>, dim3(a.num_tokens), dim3(256), 0, st, a);
  return launch_status();
}
