// Linear recurrence with a scalar decay per head and token:
//   S_t = a_t S_{t-1} + b_t k_t v_t^T,   out_t = S_t^T q_t + skip_h v_t
// the state fp32 and carried per sequence.  Retention (a constant per head) and the state-space duality form of Mamba-2
// (a_t = exp(-exp(A) dt_t), b_t = dt_t, q = C, k = B shared by a group of heads, skip = D).  Beside the lightning attention
// (lightning.hip), whose decay is a constant and whose inputs pass a silu on the way in.
#include "act_types.h"

namespace hymeta {

namespace {

// Exact exp2 for the fp32 path (the hardware's exp2 is about 1 ulp; both are far inside the state's own rounding, but the
// fp32 path is held to fp32 library functions throughout).
template <typename A>
__device__ __forceinline__ float decay_at(const hymeta_decay_scan_args& a, int64_t t, int h, float constant) {
  if (!a.log2_decay) return constant;
  const float l = a.log2_decay[t * a.num_heads + h];
  return A::kDtype == HYMETA_F32 ? exp2f(l) : __builtin_amdgcn_exp2f(l);
}

// Token by token.  grid = (heads, sequences, value columns in runs of 256); a thread owns one value column c and keeps
// that column of the state, S[:, c], in registers; q_t and k_t go through LDS.
template <typename A, int DMAX>
__global__ __launch_bounds__(256) void decay_scan_rows_kernel(hymeta_decay_scan_args a, int min_rows, int max_rows) {
  typedef typename A::elem elem;
  __shared__ float s_q[2][DMAX], s_k[2][DMAX];
  const int h = blockIdx.x, s = blockIdx.y;
  const int c = blockIdx.z * 256 + threadIdx.x;
  const int H = a.num_heads, D = a.head_dim, Dv = a.v_dim;
  const int g = h / (H / a.num_qk_heads);
  const int r0 = a.query_start_loc[s], r1 = a.query_start_loc[s + 1];
  if (r1 - r0 < min_rows || r1 - r0 > max_rows) return;
  const int slot = a.slot_idx[s];
  const bool live = c < Dv;
  float* st = (slot >= 0) ? a.state + ((static_cast<int64_t>(slot) * H + h) * D) * Dv : nullptr;
  float S[DMAX];
  const bool carry = st != nullptr && a.context_lens[s] > 0 && live;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) S[d] = (carry && d < D) ? st[static_cast<int64_t>(d) * Dv + c] : 0.f;
  const float constant = a.decay ? a.decay[h] : 1.f;
  const float skip = a.skip ? a.skip[h] : 0.f;
  for (int t = r0; t < r1; ++t) {
    const elem* q = static_cast<const elem*>(a.q) + static_cast<int64_t>(t) * a.q_stride_t + static_cast<int64_t>(g) * D;
    const elem* k = static_cast<const elem*>(a.k) + static_cast<int64_t>(t) * a.k_stride_t + static_cast<int64_t>(g) * D;
    const int buf = (t - r0) & 1;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
      s_q[buf][d] = A::ld(q + d);
      s_k[buf][d] = A::ld(k + d);
    }
    const float v = live ? A::ld(static_cast<const elem*>(a.v) + static_cast<int64_t>(t) * a.v_stride_t + static_cast<int64_t>(h) * Dv + c) : 0.f;
    const float decay = decay_at<A>(a, t, h, constant);
    const float bv = (a.v_scale ? a.v_scale[static_cast<int64_t>(t) * H + h] : 1.f) * v;
    __syncthreads();           // one barrier per token: the next token fills the other buffer
    float o = skip * v;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < D) {
        S[d] = fmaf(decay, S[d], s_k[buf][d] * bv);
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

// Sequences with one row (decode).  grid = (heads, sequences), 256 threads over the state in fours of value columns: a
// thread takes the columns 4 c4 .. 4 c4 + 3 of the rows d0, d0 + dstep, ... of S (16-byte loads and stores, four rows in
// flight together), the partial outputs of the dstep row groups meet in LDS.
constexpr int kStepMaxD = 256;
template <typename A>
__global__ __launch_bounds__(256) void decay_scan_step_kernel(hymeta_decay_scan_args a) {
  typedef typename A::elem elem;
  __shared__ float s_q[kStepMaxD], s_k[kStepMaxD];
  __shared__ __attribute__((aligned(16))) float s_o[256 * 4];
  const int h = blockIdx.x, s = blockIdx.y;
  const int t = a.query_start_loc[s];
  if (a.query_start_loc[s + 1] - t != 1) return;
  const int H = a.num_heads, D = a.head_dim, Dv = a.v_dim, Dv4 = Dv / 4;
  const int g = h / (H / a.num_qk_heads);
  const int c4 = threadIdx.x % Dv4, d0 = threadIdx.x / Dv4, dstep = 256 / Dv4;
  const int slot = a.slot_idx[s];
  float* st = slot >= 0 ? a.state + ((static_cast<int64_t>(slot) * H + h) * D) * Dv : nullptr;
  const bool carry = st != nullptr && a.context_lens[s] > 0;
  const elem* q = static_cast<const elem*>(a.q) + static_cast<int64_t>(t) * a.q_stride_t + static_cast<int64_t>(g) * D;
  const elem* k = static_cast<const elem*>(a.k) + static_cast<int64_t>(t) * a.k_stride_t + static_cast<int64_t>(g) * D;
  for (int d = threadIdx.x; d < D; d += 256) {
    s_q[d] = A::ld(q + d);
    s_k[d] = A::ld(k + d);
  }
  float v[4], bv[4];
  A::ld4(static_cast<const elem*>(a.v) + static_cast<int64_t>(t) * a.v_stride_t + static_cast<int64_t>(h) * Dv + 4 * c4, v);
  const float decay = decay_at<A>(a, t, h, a.decay ? a.decay[h] : 1.f);
  const float b = a.v_scale ? a.v_scale[static_cast<int64_t>(t) * H + h] : 1.f;
#pragma unroll
  for (int e = 0; e < 4; ++e) bv[e] = b * v[e];
  __syncthreads();
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int db = d0; db < D; db += 4 * dstep) {
    f32x4 S[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int d = db + u * dstep;
      S[u] = (carry && d < D) ? *reinterpret_cast<const f32x4*>(st + static_cast<int64_t>(d) * Dv + 4 * c4) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int d = db + u * dstep;
      if (d >= D) continue;
      const float kd = s_k[d], qd = s_q[d];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        S[u][e] = fmaf(decay, S[u][e], kd * bv[e]);
        acc[e] = fmaf(S[u][e], qd, acc[e]);
      }
      if (st != nullptr) *reinterpret_cast<f32x4*>(st + static_cast<int64_t>(d) * Dv + 4 * c4) = S[u];
    }
  }
  *reinterpret_cast<f32x4*>(&s_o[threadIdx.x * 4]) = acc;          // [d0][4 c4 + e]
  __syncthreads();
  const float skip = a.skip ? a.skip[h] : 0.f;
  for (int c = threadIdx.x; c < Dv; c += 256) {
    float o = 0.f;
    for (int gg = 0; gg < dstep; ++gg) o += s_o[(gg * Dv4 + c / 4) * 4 + (c & 3)];
    const float vc = A::ld(static_cast<const elem*>(a.v) + static_cast<int64_t>(t) * a.v_stride_t + static_cast<int64_t>(h) * Dv + c);
    a.out[static_cast<int64_t>(t) * H * Dv + static_cast<int64_t>(h) * Dv + c] = fmaf(skip, vc, o);
  }
}

inline bool step_shape(const hymeta_decay_scan_args& a) {
  const int dv4 = a.v_dim / 4;
  const int bytes = a.act_dtype == HYMETA_BF16 ? 2 : 4;
  return a.v_dim % 4 == 0 && dv4 <= 256 && 256 % dv4 == 0 && a.head_dim <= kStepMaxD && reinterpret_cast<uintptr_t>(a.state) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(a.v) % (4 * bytes) == 0 && a.v_stride_t % 4 == 0;
}

template <typename A>
void launch_rows(const hymeta_decay_scan_args& a, hipStream_t st, int min_rows, int max_rows) {
  const dim3 grid(a.num_heads, a.num_seqs, (a.v_dim + 255) / 256);
  const dim3 block(a.v_dim >= 256 ? 256 : (a.v_dim + 63) / 64 * 64);
  if (a.head_dim <= 32) hipLaunchKernelGGL((decay_scan_rows_kernel<A, 32>), grid, block, 0, st, a, min_rows, max_rows);
  else if (a.head_dim <= 64) hipLaunchKernelGGL((decay_scan_rows_kernel<A, 64>), grid, block, 0, st, a, min_rows, max_rows);
  else if (a.head_dim <= 128) hipLaunchKernelGGL((decay_scan_rows_kernel<A, 128>), grid, block, 0, st, a, min_rows, max_rows);
  else hipLaunchKernelGGL((decay_scan_rows_kernel<A, 256>), grid, block, 0, st, a, min_rows, max_rows);
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_decay_scan(const hymeta_decay_scan_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_decay_scan_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.num_heads <= 0 || a.num_qk_heads <= 0 || a.head_dim <= 0 || a.v_dim <= 0) return HYMETA_ERR_INVALID_ARG;
  if (a.num_heads % a.num_qk_heads != 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.head_dim > 256 || a.num_seqs > 65535 || a.v_dim > 256 * 65535) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.q || !a.k || !a.v || !a.state || !a.out || !a.query_start_loc || !a.context_lens || !a.slot_idx) return HYMETA_ERR_INVALID_ARG;
  if (!a.decay && !a.log2_decay) return HYMETA_ERR_INVALID_ARG;
  const int64_t qk = static_cast<int64_t>(a.num_qk_heads) * a.head_dim;
  if (a.q_stride_t < qk || a.k_stride_t < qk || a.v_stride_t < static_cast<int64_t>(a.num_heads) * a.v_dim) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  int max_rows = 0x7fffffff;
  int min_rows = 1;
  if (step_shape(a)) {
    const dim3 grid(a.num_heads, a.num_seqs);
    if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(decay_scan_step_kernel<ActBf16>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(decay_scan_step_kernel<ActF32>, grid, dim3(256), 0, st, a);
    min_rows = 2;
  }
  if (a.max_query_len >= min_rows && max_rows >= min_rows) {
    if (a.act_dtype == HYMETA_BF16) launch_rows<ActBf16>(a, st, min_rows, max_rows);
    else launch_rows<ActF32>(a, st, min_rows, max_rows);
  }
  return launch_status();
}
