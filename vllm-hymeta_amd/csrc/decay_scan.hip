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

// ------------------------------------------------------------------------------------------------
// bf16 portions in chunks of 64 rows on the matrix cores.  With S the state before the chunk, i and j rows of the
// chunk, n its number of rows, l_j the log2 decays and c_i = l_0 + ... + l_i their running sums:
//   o_i   = 2^(c_i) S^T q_i + sum_{j <= i} 2^(c_i - c_j) b_j (q_i . k_j) v_j + skip v_i
//   S_new = 2^(c_{n-1}) S + sum_j 2^(c_{n-1} - c_j) b_j k_j v_j^T
// grid = (heads, sequences, value columns in slices of 32); 4 waves, each with 16 rows of the chunk.  The state
// slice stays fp32 in registers, transposed (S^T [c][d]: a lane holds 4 value columns of one d), 16 x 16 blocks dealt
// over the waves; what enters a matrix product from fp32 (the decayed weights, the decayed keys, the state) goes in as
// hi + lo bf16 parts, two products, so that it keeps 16 bits of mantissa.  Every wave keeps the chunk's running sums in
// its lanes (lane = row of the chunk), so the decays cost shuffles and no LDS.
// ------------------------------------------------------------------------------------------------
typedef float f32x4v __attribute__((ext_vector_type(4)));
constexpr int kChunk = HYMETA_SCAN_CHUNK, kSliceV = 32;
constexpr int kChunkMinRows = 8;            // shorter portions go token by token
// Steps with a portion of kSegmentMinRows or more are cut into segments of kSegmentRows that run side by side: every
// segment but the last is summarised from a zero state (its state and the sum of its log2 decays), the summaries are chained
// into the states in front of the segments, then every segment runs from its state (three launches; a sequence's chunks
// otherwise follow each other in one workgroup per head and value slice, which leaves most of the chip idle under a single
// long prompt).
constexpr int kSegmentRows = 1024, kSegmentMinRows = 2048;
enum ChunkMode { kWhole = 0, kSummarise = 1, kApply = 2 };
constexpr float kMinLog2 = -1.0e4f;         // a decay of 0 (or an overflowed step size): finite, so that differences of sums stay numbers

__device__ __forceinline__ f32x4v mfma16(bf16x8 a, bf16x8 b, f32x4v c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }

template <int D>
__global__ __launch_bounds__(256) void decay_scan_chunk_kernel(hymeta_decay_scan_args a, int min_rows, int seg_rows, int nseg, int mode) {
  constexpr int PK = D + 8, PT = kChunk + 8, NBW = (2 * D / 16) / 4;
  __shared__ __attribute__((aligned(16))) uint16_t sk[kChunk * PK];          // k, a row per key
  __shared__ __attribute__((aligned(16))) uint16_t skt[2][D * PT];           // decayed keys, transposed [d][key], hi / lo
  __shared__ __attribute__((aligned(16))) uint16_t svt[kSliceV * PT];        // v of the slice, transposed [c][key]
  __shared__ __attribute__((aligned(16))) uint16_t sst[2][kSliceV * PK];     // state^T [c][d], hi / lo
  const int h = blockIdx.x, s = blockIdx.y / nseg, seg = blockIdx.y % nseg, vs = blockIdx.z;
  const int r0 = a.query_start_loc[s], rows_all = a.query_start_loc[s + 1] - r0;
  if (rows_all < min_rows) return;
  // this workgroup's rows of the portion: all of them (kWhole), or one segment
  const int r_lo = mode == kWhole ? 0 : seg * seg_rows;
  if (r_lo >= rows_all) return;
  const int rows = mode == kWhole ? rows_all : min(rows_all, r_lo + seg_rows);        // (end of the rows, not their count)
  const bool last = rows == rows_all;
  if (mode == kSummarise && last) return;                    // nothing comes behind the last segment
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 15, g4 = lane >> 4;
  const int H = a.num_heads, Dv = a.v_dim;
  const int g = h / (H / a.num_qk_heads);
  const int slot = a.slot_idx[s];
  float* st = slot >= 0 ? a.state + ((static_cast<int64_t>(slot) * H + h) * D) * Dv + vs * kSliceV : nullptr;
  const float l2_const = a.decay ? fmaxf(a.decay[h] > 0.f ? log2f(a.decay[h]) : -INFINITY, kMinLog2) : 0.f;
  const float skip = a.skip ? a.skip[h] : 0.f;
  const bool carry = st != nullptr && a.context_lens[s] > 0;
  // a segment's place in the workspace: its summary (kSummarise writes it), then the state in front of it (kApply reads it);
  // the segments' sums of log2 decays lie behind all the states
  const int64_t seg_at = (static_cast<int64_t>(s) * nseg + seg) * H + h;
  float* wsp = mode == kWhole ? nullptr : static_cast<float*>(a.workspace) + (seg_at * D) * Dv + vs * kSliceV;
  const float* init = mode == kWhole ? (carry ? st : nullptr) : mode == kApply ? wsp : nullptr;
  f32x4v S[NBW];
#pragma unroll
  for (int ib = 0; ib < NBW; ++ib) {
    const int b = wave + 4 * ib, cb = b & 1, db = b >> 1;
    S[ib] = init ? *reinterpret_cast<const f32x4v*>(init + static_cast<int64_t>(16 * db + n) * Dv + 16 * cb + 4 * g4) : f32x4v{0.f, 0.f, 0.f, 0.f};
  }
  float seg_total = 0.f;
  auto state_to_lds = [&]() {
#pragma unroll
    for (int ib = 0; ib < NBW; ++ib) {
      const int b = wave + 4 * ib, cb = b & 1, db = b >> 1;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float v = S[ib][r];
        const uint16_t hi = f2bf(v);
        const int at = (16 * cb + 4 * g4 + r) * PK + 16 * db + n;
        sst[0][at] = hi;
        sst[1][at] = f2bf(v - bf2f(hi));
      }
    }
  };
  state_to_lds();
  const uint16_t* qp = static_cast<const uint16_t*>(a.q) + static_cast<int64_t>(g) * D;
  const uint16_t* kp = static_cast<const uint16_t*>(a.k) + static_cast<int64_t>(g) * D;
  const uint16_t* vp = static_cast<const uint16_t*>(a.v) + static_cast<int64_t>(h) * Dv + vs * kSliceV;
  // the rows of a chunk as they come from memory: this thread's share of the keys (KPT groups of 8 columns of one row) and
  // of the value slice, this lane's query fragment, and row `lane`'s log2 decay and input weight; loaded a chunk ahead
  constexpr int KPT = kChunk * (D / 8) / 256;
  u32x4 rk[KPT], rv, rq[D / 32];
  float rl, rb;
  auto fetch = [&](int c0) {
    const int nrow = min(kChunk, rows - c0);
    const int64_t t0 = r0 + c0;
#pragma unroll
    for (int u = 0; u < KPT; ++u) {
      const int idx = tid + 256 * u, j = idx % kChunk, ch = idx / kChunk;
      rk[u] = u32x4{0u, 0u, 0u, 0u};
      if (j < nrow) rk[u] = ld16g(kp + (t0 + j) * a.k_stride_t + 8 * ch);
    }
    {
      const int j = tid % kChunk, ch = tid / kChunk;
      rv = u32x4{0u, 0u, 0u, 0u};
      if (j < nrow) rv = ld16g(vp + (t0 + j) * a.v_stride_t + 8 * ch);
    }
    const int i = 16 * wave + n;
#pragma unroll
    for (int sd = 0; sd < D / 32; ++sd) {
      rq[sd] = u32x4{0u, 0u, 0u, 0u};
      if (i < nrow && mode != kSummarise) rq[sd] = ld16g(qp + (t0 + i) * a.q_stride_t + 32 * sd + 8 * g4);
    }
    rl = 0.f, rb = 0.f;
    if (lane < nrow) {
      rl = a.log2_decay ? fmaxf(a.log2_decay[(t0 + lane) * H + h], kMinLog2) : l2_const;
      rb = a.v_scale ? a.v_scale[(t0 + lane) * H + h] : 1.f;
    }
  };
  static_assert(kChunk * (kSliceV / 8) == 256, "one group of the value slice per thread");
  fetch(r_lo);
  for (int c0 = r_lo; c0 < rows; c0 += kChunk) {
    const int nrow = min(kChunk, rows - c0);
    // running sums of the chunk's log2 decays over the wave's lanes (rows past the portion add 0)
    float cum = rl;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float up = __shfl_up(cum, o, 64);
      if (lane >= o) cum += up;
    }
    const float total = __shfl(cum, nrow - 1, 64);
    seg_total += total;
    const float bw = rb;
    // a wave's lanes hold 64 different rows of one 8-column group (row = lane): the transposed 2-byte stores of a wave fall
    // on consecutive addresses, the row-major 16-byte stores on different banks
    const float kd = lane < nrow ? __builtin_amdgcn_exp2f(total - cum) * bw : 0.f;
#pragma unroll
    for (int u = 0; u < KPT; ++u) {
      const int idx = tid + 256 * u, j = idx % kChunk, ch = idx / kChunk;
      st16(&sk[j * PK + 8 * ch], rk[u]);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t w = rk[u][e >> 1];
        const float x = (e & 1 ? hi_bf(w) : lo_bf(w)) * kd;
        const uint16_t hi = f2bf(x);
        skt[0][(8 * ch + e) * PT + j] = hi;
        skt[1][(8 * ch + e) * PT + j] = f2bf(x - bf2f(hi));
      }
    }
    {
      const int j = tid % kChunk, ch = tid / kChunk;
#pragma unroll
      for (int e = 0; e < 8; ++e) svt[(8 * ch + e) * PT + j] = static_cast<uint16_t>(e & 1 ? rv[e >> 1] >> 16 : rv[e >> 1] & 0xffffu);
    }
    const int i = 16 * wave + n;                       // this lane's row of the chunk (as a column of the products)
    bf16x8 q[D / 32];
#pragma unroll
    for (int sd = 0; sd < D / 32; ++sd) q[sd] = __builtin_bit_cast(bf16x8, rq[sd]);
    __syncthreads();
    if (c0 + kChunk < rows) fetch(c0 + kChunk);        // in flight while this chunk is multiplied
    if (mode != kSummarise) {
      // weights of the chunk's own rows: (q_i . k_j) 2^(c_i - c_j) b_j for j <= i, as hi + lo parts
      const float cum_i = __shfl(cum, i, 64);
      uint32_t phi[4][2], plo[4][2];
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        f32x4v sc = f32x4v{0.f, 0.f, 0.f, 0.f};
        if (ks <= wave) {
#pragma unroll
          for (int sd = 0; sd < D / 32; ++sd)
            sc = mfma16(__builtin_bit_cast(bf16x8, ld16(&sk[(16 * ks + n) * PK + 32 * sd + 8 * g4])), q[sd], sc);
        }
        float p[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int j = 16 * ks + 4 * g4 + r;
          const float cum_j = __shfl(cum, j, 64), b_j = __shfl(bw, j, 64);
          p[r] = (ks <= wave && j <= i) ? sc[r] * __builtin_amdgcn_exp2f(cum_i - cum_j) * b_j : 0.f;
        }
#pragma unroll
        for (int r2 = 0; r2 < 2; ++r2) {
          const uint32_t hi = pack_bf16x2(p[2 * r2], p[2 * r2 + 1]);
          phi[ks][r2] = hi;
          plo[ks][r2] = pack_bf16x2(p[2 * r2] - lo_bf(hi), p[2 * r2 + 1] - hi_bf(hi));
        }
      }
      f32x4v o[2];
      const float row_decay = __builtin_amdgcn_exp2f(cum_i);
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
        // the state before the chunk
        f32x4v x = f32x4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sd = 0; sd < D / 32; ++sd) {
          x = mfma16(__builtin_bit_cast(bf16x8, ld16(&sst[0][(16 * cb + n) * PK + 32 * sd + 8 * g4])), q[sd], x);
          x = mfma16(__builtin_bit_cast(bf16x8, ld16(&sst[1][(16 * cb + n) * PK + 32 * sd + 8 * g4])), q[sd], x);
        }
        f32x4v acc = x * row_decay;
        if (skip != 0.f) {
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[r] = fmaf(skip, bf2f(svt[(16 * cb + 4 * g4 + r) * PT + i]), acc[r]);
        }
#pragma unroll
        for (int kp2 = 0; kp2 < 2; ++kp2) {
          if (2 * kp2 > wave) continue;
          // k index 8 g4 + e of the product: keys 32 kp2 + 4 g4 + e for e < 4, 32 kp2 + 16 + 4 g4 + e - 4 after
          const u32x2 v0 = *reinterpret_cast<const u32x2*>(&svt[(16 * cb + n) * PT + 32 * kp2 + 4 * g4]);
          const u32x2 v1 = *reinterpret_cast<const u32x2*>(&svt[(16 * cb + n) * PT + 32 * kp2 + 16 + 4 * g4]);
          const bf16x8 vf = __builtin_bit_cast(bf16x8, (u32x4{v0[0], v0[1], v1[0], v1[1]}));
          acc = mfma16(vf, __builtin_bit_cast(bf16x8, (u32x4{phi[2 * kp2][0], phi[2 * kp2][1], phi[2 * kp2 + 1][0], phi[2 * kp2 + 1][1]})), acc);
          acc = mfma16(vf, __builtin_bit_cast(bf16x8, (u32x4{plo[2 * kp2][0], plo[2 * kp2][1], plo[2 * kp2 + 1][0], plo[2 * kp2 + 1][1]})), acc);
        }
        o[cb] = acc;
      }
      if (i < nrow) {
        float* orow = a.out + static_cast<int64_t>(r0 + c0 + i) * H * Dv + static_cast<int64_t>(h) * Dv + vs * kSliceV;
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) *reinterpret_cast<f32x4v*>(orow + 16 * cb + 4 * g4) = o[cb];
      }
    }
    // the state after the chunk
    const float chunk_decay = __builtin_amdgcn_exp2f(total);
#pragma unroll
    for (int ib = 0; ib < NBW; ++ib) {
      const int b = wave + 4 * ib, cb = b & 1, db = b >> 1;
      f32x4v acc = S[ib] * chunk_decay;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const bf16x8 vf = __builtin_bit_cast(bf16x8, ld16(&svt[(16 * cb + n) * PT + 32 * kk + 8 * g4]));
        acc = mfma16(vf, __builtin_bit_cast(bf16x8, ld16(&skt[0][(16 * db + n) * PT + 32 * kk + 8 * g4])), acc);
        acc = mfma16(vf, __builtin_bit_cast(bf16x8, ld16(&skt[1][(16 * db + n) * PT + 32 * kk + 8 * g4])), acc);
      }
      S[ib] = acc;
    }
    __syncthreads();            // every wave is done with this chunk's tiles and with the old state's image
    state_to_lds();             // (made visible by the barrier after the next chunk's staging)
  }
  float* to = mode == kSummarise ? wsp : (last ? st : nullptr);
  if (to != nullptr) {
#pragma unroll
    for (int ib = 0; ib < NBW; ++ib) {
      const int b = wave + 4 * ib, cb = b & 1, db = b >> 1;
      *reinterpret_cast<f32x4v*>(to + static_cast<int64_t>(16 * db + n) * Dv + 16 * cb + 4 * g4) = S[ib];
    }
  }
  if (mode == kSummarise && vs == 0 && tid == 0) {
    float* totals = static_cast<float*>(a.workspace) + static_cast<int64_t>(a.num_seqs) * nseg * H * D * Dv;
    totals[seg_at] = seg_total;
  }
}

// The segments' summaries (each segment's state had it started from zero) become the states in front of the segments:
// run = carried state; per segment: place <- run, run <- 2^(segment's sum of log2 decays) run + summary.  An element per thread.
__global__ __launch_bounds__(256) void decay_scan_chain_kernel(hymeta_decay_scan_args a, int min_rows, int seg_rows, int nseg) {
  const int s = blockIdx.y;
  const int rows = a.query_start_loc[s + 1] - a.query_start_loc[s];
  if (rows < min_rows) return;
  const int64_t per_head = static_cast<int64_t>(a.head_dim) * a.v_dim, per_seq = per_head * a.num_heads;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= per_seq) return;
  const int h = static_cast<int>(idx / per_head);
  const int slot = a.slot_idx[s];
  float run = (slot >= 0 && a.context_lens[s] > 0) ? a.state[static_cast<int64_t>(slot) * per_seq + idx] : 0.f;
  const int segs = (rows + seg_rows - 1) / seg_rows;
  float* p = static_cast<float*>(a.workspace) + static_cast<int64_t>(s) * nseg * per_seq + idx;
  const float* totals = static_cast<const float*>(a.workspace) + static_cast<int64_t>(a.num_seqs) * nseg * per_seq +
                        static_cast<int64_t>(s) * nseg * a.num_heads + h;
  for (int seg = 0; seg < segs; ++seg, p += per_seq) {
    const bool more = seg < segs - 1;
    const float summary = more ? *p : 0.f;
    *p = run;
    if (more) run = __builtin_amdgcn_exp2f(totals[static_cast<int64_t>(seg) * a.num_heads]) * run + summary;
  }
}

inline bool chunk_shape(const hymeta_decay_scan_args& a) {
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  return a.act_dtype == HYMETA_BF16 && (a.head_dim == 32 || a.head_dim == 64 || a.head_dim == 128) && a.v_dim % kSliceV == 0 &&
         a.q_stride_t % 8 == 0 && a.k_stride_t % 8 == 0 && a.v_stride_t % 8 == 0 && aligned(a.q) && aligned(a.k) && aligned(a.v) &&
         aligned(a.state) && aligned(a.out) && a.v_dim / kSliceV <= 65535;
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

extern "C" size_t hymeta_decay_scan_workspace_bytes(int32_t num_seqs, int32_t num_heads, int32_t head_dim, int32_t v_dim, int32_t max_query_len) {
  if (num_seqs <= 0 || num_heads <= 0 || head_dim <= 0 || v_dim <= 0 || max_query_len < kSegmentMinRows) return 0;
  const size_t nseg = (static_cast<size_t>(max_query_len) + kSegmentRows - 1) / kSegmentRows;
  return nseg * num_seqs * num_heads * (static_cast<size_t>(head_dim) * v_dim + 1) * sizeof(float);
}

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
  if (chunk_shape(a) && a.max_query_len >= kChunkMinRows) {
    const size_t need = hymeta_decay_scan_workspace_bytes(a.num_seqs, a.num_heads, a.head_dim, a.v_dim, a.max_query_len);
    const int nseg = need > 0 ? (a.max_query_len + kSegmentRows - 1) / kSegmentRows : 1;
    if (need > 0 && (!a.workspace || a.workspace_bytes < need)) return HYMETA_ERR_WORKSPACE;
    if (static_cast<int64_t>(a.num_seqs) * nseg > 65535) return HYMETA_ERR_UNSUPPORTED;
    const dim3 grid(a.num_heads, a.num_seqs * nseg, a.v_dim / kSliceV);
    auto chunks = [&](int mode) {
      if (a.head_dim == 32) hipLaunchKernelGGL(decay_scan_chunk_kernel<32>, grid, dim3(256), 0, st, a, kChunkMinRows, kSegmentRows, nseg, mode);
      else if (a.head_dim == 64) hipLaunchKernelGGL(decay_scan_chunk_kernel<64>, grid, dim3(256), 0, st, a, kChunkMinRows, kSegmentRows, nseg, mode);
      else hipLaunchKernelGGL(decay_scan_chunk_kernel<128>, grid, dim3(256), 0, st, a, kChunkMinRows, kSegmentRows, nseg, mode);
    };
    if (nseg == 1) {
      chunks(kWhole);
    } else {
      chunks(kSummarise);
      const int64_t per_seq = static_cast<int64_t>(a.num_heads) * a.head_dim * a.v_dim;
      hipLaunchKernelGGL(decay_scan_chain_kernel, dim3(static_cast<unsigned>((per_seq + 255) / 256), a.num_seqs), dim3(256), 0, st, a, kChunkMinRows,
                         kSegmentRows, nseg);
      chunks(kApply);
    }
    max_rows = kChunkMinRows - 1;
  }
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
