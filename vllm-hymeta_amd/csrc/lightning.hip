// Linear attention with a constant decay per head ("lightning attention"): S <- decay S + k v^T, out = S^T q, the state
// fp32 and carried per sequence; and the output norm with its sigmoid gate.
#include "act_types.h"

namespace hymeta {

namespace {

__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }

// Token by token.  grid = (heads, sequences, value columns in runs of 256); a thread owns one value column c and keeps
// that column of the state, S[:, c], in registers; q_t and k_t go through LDS.
template <typename A, int DMAX>
__global__ __launch_bounds__(256) void lightning_rows_kernel(hymeta_lightning_attention_args a, int min_rows, int max_rows) {
  typedef typename A::elem elem;
  __shared__ float s_q[2][DMAX], s_k[2][DMAX];
  const int h = blockIdx.x, s = blockIdx.y;
  const int c = blockIdx.z * 256 + threadIdx.x;
  const int H = a.num_heads, D = a.head_dim, Dv = a.v_dim;
  const int r0 = a.query_start_loc[s], r1 = a.query_start_loc[s + 1];
  if (r1 - r0 < min_rows || r1 - r0 > max_rows) return;          // single rows / longer portions: the other kernels'
  const int slot = a.slot_idx[s];
  const bool live = c < Dv;
  float* st = (slot >= 0) ? a.state + ((static_cast<int64_t>(slot) * H + h) * D) * Dv : nullptr;
  float S[DMAX];
  const bool carry = st != nullptr && a.context_lens[s] > 0 && live;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) S[d] = (carry && d < D) ? st[static_cast<int64_t>(d) * Dv + c] : 0.f;
  const float decay = a.decay[h];
  const int64_t q_off = static_cast<int64_t>(h) * D, k_off = static_cast<int64_t>(H) * D + q_off;
  const int64_t v_off = 2 * static_cast<int64_t>(H) * D + static_cast<int64_t>(h) * Dv;
  for (int t = r0; t < r1; ++t) {
    const elem* row = static_cast<const elem*>(a.qkv) + static_cast<int64_t>(t) * a.qkv_stride_t;
    const int buf = (t - r0) & 1;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
      s_q[buf][d] = silu_f(A::ld(row + q_off + d));
      s_k[buf][d] = silu_f(A::ld(row + k_off + d));
    }
    const float v = live ? silu_f(A::ld(row + v_off + c)) : 0.f;
    __syncthreads();           // one barrier per token: the next token fills the other buffer
    float o = 0.f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < D) {
        S[d] = fmaf(decay, S[d], s_k[buf][d] * v);
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

// Rows of up to kGatedCached columns are read once (a thread keeps its columns in registers).
constexpr int kGatedPerThread = 16, kGatedCached = 256 * kGatedPerThread;

// grid = (rows, groups): a workgroup norms one of the row's equal consecutive parts.
template <typename A, bool Cached>
__global__ __launch_bounds__(256) void gated_rms_norm_kernel(hymeta_gated_rms_norm_args a) {
  typedef typename A::elem elem;
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int width = a.width / gridDim.y, c0 = blockIdx.y * width;
  const float* x = a.x + t * a.width + c0;
  const elem* g = static_cast<const elem*>(a.gate) + t * a.gate_stride_t + c0;
  const float* weight = a.weight ? a.weight + c0 : nullptr;
  elem* out = static_cast<elem*>(a.out) + t * a.width + c0;
  const bool silu = a.gate_act == HYMETA_GATE_SILU, first = a.gate_first != 0;
  auto gate_of = [&](float gv) { const float sg = sigmoid_exact(gv); return silu ? gv * sg : sg; };
  float ss = 0.f;
  if (Cached) {
    float xv[kGatedPerThread], gv[kGatedPerThread];
#pragma unroll
    for (int u = 0; u < kGatedPerThread; ++u) {
      const int c = threadIdx.x + 256 * u;
      xv[u] = c < width ? x[c] : 0.f;
      gv[u] = c < width ? gate_of(A::ld(g + c)) : 0.f;
      if (first) xv[u] *= gv[u], gv[u] = 1.f;
      ss = fmaf(xv[u], xv[u], ss);
    }
    ss = block_sum<4>(ss, red);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(width) + a.eps);
#pragma unroll
    for (int u = 0; u < kGatedPerThread; ++u) {
      const int c = threadIdx.x + 256 * u;
      if (c < width) A::st(out + c, xv[u] * inv * (weight ? weight[c] : 1.f) * gv[u]);
    }
    return;
  }
  for (int c = threadIdx.x; c < width; c += 256) {
    const float v = first ? x[c] * gate_of(A::ld(g + c)) : x[c];
    ss = fmaf(v, v, ss);
  }
  ss = block_sum<4>(ss, red);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(width) + a.eps);
  for (int c = threadIdx.x; c < width; c += 256) {
    const float gv = gate_of(A::ld(g + c));
    A::st(out + c, x[c] * inv * (weight ? weight[c] : 1.f) * gv);
  }
}

// Narrow groups (a head's output): a wave per (row, group), the group's columns in the lanes' registers, no barrier.
constexpr int kGatedWavePerLane = 16, kGatedWaveCols = 64 * kGatedWavePerLane;

template <typename A>
__global__ __launch_bounds__(256) void gated_rms_norm_wave_kernel(hymeta_gated_rms_norm_args a, int groups) {
  typedef typename A::elem elem;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, grp = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (grp >= groups) return;
  const int width = a.width / groups, c0 = grp * width;
  const float* x = a.x + t * a.width + c0;
  const elem* g = static_cast<const elem*>(a.gate) + t * a.gate_stride_t + c0;
  const float* weight = a.weight ? a.weight + c0 : nullptr;
  elem* out = static_cast<elem*>(a.out) + t * a.width + c0;
  const bool silu = a.gate_act == HYMETA_GATE_SILU, first = a.gate_first != 0;
  float xv[kGatedWavePerLane], gv[kGatedWavePerLane];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < kGatedWavePerLane; ++u) {
    const int c = lane + 64 * u;
    if (64 * u >= width) { xv[u] = 0.f, gv[u] = 0.f; continue; }
    xv[u] = c < width ? x[c] : 0.f;
    const float raw = c < width ? A::ld(g + c) : 0.f;
    const float sg = sigmoid_exact(raw);
    gv[u] = silu ? raw * sg : sg;
    if (first) xv[u] *= gv[u], gv[u] = 1.f;
    ss = fmaf(xv[u], xv[u], ss);
  }
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(width) + a.eps);
#pragma unroll
  for (int u = 0; u < kGatedWavePerLane; ++u) {
    const int c = lane + 64 * u;
    if (c < width) A::st(out + c, xv[u] * inv * (weight ? weight[c] : 1.f) * gv[u]);
  }
}

// ------------------------------------------------------------------------------------------------
// bf16 portions in chunks of 64 rows on the matrix cores.  With S the state before the chunk, i and j rows of the
// chunk, n its number of rows and L = decay:
//   o_i   = L^(i+1) S^T q_i + sum_{j <= i} L^(i-j) (q_i . k_j) v_j
//   S_new = L^n S + sum_j L^(n-1-j) k_j v_j^T
// grid = (heads, sequences, value columns in slices of 32); 4 waves, each with 16 rows of the chunk.  The state
// slice stays fp32 in registers, transposed (S^T [c][d]: a lane holds 4 value columns of one d), 16 x 16 blocks dealt
// over the waves; what enters a matrix product from fp32 (the decayed weights, the decayed keys, the state) goes in as
// hi + lo bf16 parts, two products, so that it keeps 16 bits of mantissa.
// ------------------------------------------------------------------------------------------------
typedef float f32x4v __attribute__((ext_vector_type(4)));
constexpr int kChunk = HYMETA_LIGHTNING_CHUNK, kSliceV = 32;
constexpr int kChunkMinRows = 8;            // shorter portions go token by token
// Steps with a portion of kSegmentMinRows or more are cut into segments of kSegmentRows that run side by side: every
// segment but the last is summarised from a zero state, the summaries are chained into the states in front of the
// segments, then every segment runs from its state (three launches; a sequence's chunks otherwise follow each other in
// one workgroup per head and value slice, which leaves most of the chip idle under a single long prompt).
constexpr int kSegmentRows = 1024, kSegmentMinRows = 2048;
enum ChunkMode { kWhole = 0, kSummarise = 1, kApply = 2 };

__device__ __forceinline__ f32x4v mfma16(bf16x8 a, bf16x8 b, f32x4v c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }

__device__ __forceinline__ float decay_pow(float log2_decay, int x) {
  return x == 0 ? 1.f : __builtin_amdgcn_exp2f(static_cast<float>(x) * log2_decay);
}

// the hardware's exponential and reciprocal (about 1 ulp each): the inputs and the result are bf16
__device__ __forceinline__ float silu_fast(float x) { return x * __builtin_amdgcn_rcpf(1.f + __expf(-x)); }

// 8 bf16 of a row through silu, back to bf16 (and, optionally, the fp32 values)
__device__ __forceinline__ u32x4 silu8(u32x4 raw, float* vals) {
  u32x4 out;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float lo = silu_fast(bf2f(static_cast<uint16_t>(raw[e] & 0xffffu))), hi = silu_fast(bf2f(static_cast<uint16_t>(raw[e] >> 16)));
    if (vals) vals[2 * e] = lo, vals[2 * e + 1] = hi;
    out[e] = pack_bf16x2(lo, hi);
  }
  return out;
}

template <int D>
__global__ __launch_bounds__(256) void lightning_chunk_kernel(hymeta_lightning_attention_args a, int min_rows, int seg_rows, int nseg, int mode) {
  constexpr int PK = D + 8, PT = kChunk + 8, NBW = (2 * D / 16) / 4;
  __shared__ __attribute__((aligned(16))) uint16_t sk[kChunk * PK];          // silu(k), a row per key
  __shared__ __attribute__((aligned(16))) uint16_t skt[2][D * PT];           // decayed keys, transposed [d][key], hi / lo
  __shared__ __attribute__((aligned(16))) uint16_t svt[kSliceV * PT];        // silu(v) of the slice, transposed [c][key]
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
  const int slot = a.slot_idx[s];
  float* st = slot >= 0 ? a.state + ((static_cast<int64_t>(slot) * H + h) * D) * Dv + vs * kSliceV : nullptr;
  const float decay = a.decay[h];
  const float l2 = decay > 0.f ? log2f(decay) : -INFINITY;
  const bool carry = st != nullptr && a.context_lens[s] > 0;
  // a segment's place in the workspace: its summary (kSummarise writes it), then the state in front of it (kApply reads it)
  float* wsp = mode == kWhole ? nullptr
                              : static_cast<float*>(a.workspace) + (((static_cast<int64_t>(s) * nseg + seg) * H + h) * D) * Dv + vs * kSliceV;
  const float* init = mode == kWhole ? (carry ? st : nullptr) : mode == kApply ? wsp : nullptr;
  f32x4v S[NBW];
#pragma unroll
  for (int ib = 0; ib < NBW; ++ib) {
    const int b = wave + 4 * ib, cb = b & 1, db = b >> 1;
    S[ib] = init ? *reinterpret_cast<const f32x4v*>(init + static_cast<int64_t>(16 * db + n) * Dv + 16 * cb + 4 * g4) : f32x4v{0.f, 0.f, 0.f, 0.f};
  }
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
  const uint16_t* qkv = static_cast<const uint16_t*>(a.qkv);
  const int64_t q_off = static_cast<int64_t>(h) * D, k_off = static_cast<int64_t>(H) * D + q_off;
  const int64_t v_off = 2 * static_cast<int64_t>(H) * D + static_cast<int64_t>(h) * Dv + vs * kSliceV;
  // the rows of a chunk as they come from memory: this thread's share of the keys (KPT groups of 8 columns of one row) and
  // of the value slice, and this lane's query fragment; loaded a chunk ahead
  constexpr int KPT = kChunk * (D / 8) / 256;
  u32x4 rk[KPT], rv, rq[D / 32];
  auto fetch = [&](int c0) {
    const int nrow = min(kChunk, rows - c0);
    const uint16_t* base = qkv + static_cast<int64_t>(r0 + c0) * a.qkv_stride_t;
#pragma unroll
    for (int u = 0; u < KPT; ++u) {
      const int idx = tid + 256 * u, j = idx % kChunk, ch = idx / kChunk;
      rk[u] = u32x4{0u, 0u, 0u, 0u};
      if (j < nrow) rk[u] = ld16g(base + j * a.qkv_stride_t + k_off + 8 * ch);
    }
    {
      const int j = tid % kChunk, ch = tid / kChunk;
      rv = u32x4{0u, 0u, 0u, 0u};
      if (j < nrow) rv = ld16g(base + j * a.qkv_stride_t + v_off + 8 * ch);
    }
    const int i = 16 * wave + n;
#pragma unroll
    for (int sd = 0; sd < D / 32; ++sd) {
      rq[sd] = u32x4{0u, 0u, 0u, 0u};
      if (i < nrow && mode != kSummarise) rq[sd] = ld16g(base + i * a.qkv_stride_t + q_off + 32 * sd + 8 * g4);
    }
  };
  static_assert(kChunk * (kSliceV / 8) == 256, "one group of the value slice per thread");
  fetch(r_lo);
  for (int c0 = r_lo; c0 < rows; c0 += kChunk) {
    const int nrow = min(kChunk, rows - c0);
    const uint16_t* base = qkv + static_cast<int64_t>(r0 + c0) * a.qkv_stride_t;
    (void)base;
    // a wave's lanes hold 64 different rows of one 8-column group: the transposed 2-byte stores of a wave fall on
    // consecutive addresses (a lane per key), the row-major 16-byte stores on different banks
#pragma unroll
    for (int u = 0; u < KPT; ++u) {
      const int idx = tid + 256 * u, j = idx % kChunk, ch = idx / kChunk;
      float vals[8];
      u32x4 packed = silu8(rk[u], vals);            // rows past the portion were fetched as zeros: silu(0) = 0
      st16(&sk[j * PK + 8 * ch], packed);
      const float kd = j < nrow ? decay_pow(l2, nrow - 1 - j) : 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float x = vals[e] * kd;
        const uint16_t hi = f2bf(x);
        skt[0][(8 * ch + e) * PT + j] = hi;
        skt[1][(8 * ch + e) * PT + j] = f2bf(x - bf2f(hi));
      }
    }
    {
      const int j = tid % kChunk, ch = tid / kChunk;
      const u32x4 packed = silu8(rv, nullptr);
#pragma unroll
      for (int e = 0; e < 8; ++e) svt[(8 * ch + e) * PT + j] = static_cast<uint16_t>(e & 1 ? packed[e >> 1] >> 16 : packed[e >> 1] & 0xffffu);
    }
    const int i = 16 * wave + n;                       // this lane's row of the chunk (as a column of the products)
    bf16x8 q[D / 32];
#pragma unroll
    for (int sd = 0; sd < D / 32; ++sd) q[sd] = __builtin_bit_cast(bf16x8, silu8(rq[sd], nullptr));
    __syncthreads();
    if (c0 + kChunk < rows) fetch(c0 + kChunk);        // in flight while this chunk is multiplied
    if (mode != kSummarise) {
      // weights of the chunk's own rows: (q_i . k_j) L^(i-j) for j <= i, as hi + lo parts
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
          p[r] = (ks <= wave && j <= i) ? sc[r] * decay_pow(l2, i - j) : 0.f;
        }
  #pragma unroll
        for (int r2 = 0; r2 < 2; ++r2) {
          const uint32_t hi = pack_bf16x2(p[2 * r2], p[2 * r2 + 1]);
          phi[ks][r2] = hi;
          plo[ks][r2] = pack_bf16x2(p[2 * r2] - lo_bf(hi), p[2 * r2 + 1] - hi_bf(hi));
        }
      }
      f32x4v o[2];
      const float row_decay = decay_pow(l2, i + 1);
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
  #pragma unroll
        for (int kp = 0; kp < 2; ++kp) {
          if (2 * kp > wave) continue;
          // k index 8 g4 + e of the product: keys 32 kp + 4 g4 + e for e < 4, 32 kp + 16 + 4 g4 + e - 4 after
          const u32x2 v0 = *reinterpret_cast<const u32x2*>(&svt[(16 * cb + n) * PT + 32 * kp + 4 * g4]);
          const u32x2 v1 = *reinterpret_cast<const u32x2*>(&svt[(16 * cb + n) * PT + 32 * kp + 16 + 4 * g4]);
          const bf16x8 vf = __builtin_bit_cast(bf16x8, (u32x4{v0[0], v0[1], v1[0], v1[1]}));
          acc = mfma16(vf, __builtin_bit_cast(bf16x8, (u32x4{phi[2 * kp][0], phi[2 * kp][1], phi[2 * kp + 1][0], phi[2 * kp + 1][1]})), acc);
          acc = mfma16(vf, __builtin_bit_cast(bf16x8, (u32x4{plo[2 * kp][0], plo[2 * kp][1], plo[2 * kp + 1][0], plo[2 * kp + 1][1]})), acc);
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
    const float chunk_decay = decay_pow(l2, nrow);
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
}

// The segments' summaries (each segment's state had it started from zero) become the states in front of the segments:
// run = carried state; per segment: place <- run, run <- decay^(segment's rows) run + summary.  An element per thread.
__global__ __launch_bounds__(256) void lightning_chain_kernel(hymeta_lightning_attention_args a, int min_rows, int seg_rows, int nseg) {
  const int s = blockIdx.y;
  const int rows = a.query_start_loc[s + 1] - a.query_start_loc[s];
  if (rows < min_rows) return;
  const int64_t per_head = static_cast<int64_t>(a.head_dim) * a.v_dim, per_seq = per_head * a.num_heads;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= per_seq) return;
  const int h = static_cast<int>(idx / per_head);
  const float decay = a.decay[h];
  const float l2 = decay > 0.f ? log2f(decay) : -INFINITY;
  const int slot = a.slot_idx[s];
  float run = (slot >= 0 && a.context_lens[s] > 0) ? a.state[static_cast<int64_t>(slot) * per_seq + idx] : 0.f;
  const int segs = (rows + seg_rows - 1) / seg_rows;
  float* p = static_cast<float*>(a.workspace) + static_cast<int64_t>(s) * nseg * per_seq + idx;
  for (int seg = 0; seg < segs; ++seg, p += per_seq) {
    const float summary = seg < segs - 1 ? *p : 0.f;
    *p = run;
    run = decay_pow(l2, min(seg_rows, rows - seg * seg_rows)) * run + summary;
  }
}

inline bool chunk_shape(const hymeta_lightning_attention_args& a) {
  return a.act_dtype == HYMETA_BF16 && (a.head_dim == 32 || a.head_dim == 64 || a.head_dim == 128) && a.v_dim % kSliceV == 0 &&
         a.qkv_stride_t % 8 == 0 && reinterpret_cast<uintptr_t>(a.qkv) % 16 == 0 && reinterpret_cast<uintptr_t>(a.state) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(a.out) % 16 == 0 && a.v_dim / kSliceV <= 65535;
}

// Sequences with one row (decode).  grid = (heads, sequences), 256 threads over the state in fours of value columns: a
// thread takes the columns 4 c4 .. 4 c4 + 3 of the rows d0, d0 + dstep, ... of S (16-byte loads and stores, four rows in
// flight together), the partial outputs of the dstep row groups meet in LDS.
constexpr int kStepMaxD = 256;
template <typename A>
__global__ __launch_bounds__(256) void lightning_step_kernel(hymeta_lightning_attention_args a) {
  typedef typename A::elem elem;
  __shared__ float s_q[kStepMaxD], s_k[kStepMaxD];
  __shared__ __attribute__((aligned(16))) float s_o[256 * 4];
  const int h = blockIdx.x, s = blockIdx.y;
  const int t = a.query_start_loc[s];
  if (a.query_start_loc[s + 1] - t != 1) return;
  const int H = a.num_heads, D = a.head_dim, Dv = a.v_dim, Dv4 = Dv / 4;
  const int c4 = threadIdx.x % Dv4, d0 = threadIdx.x / Dv4, dstep = 256 / Dv4;
  const int slot = a.slot_idx[s];
  float* st = slot >= 0 ? a.state + ((static_cast<int64_t>(slot) * H + h) * D) * Dv : nullptr;
  const bool carry = st != nullptr && a.context_lens[s] > 0;
  const elem* row = static_cast<const elem*>(a.qkv) + static_cast<int64_t>(t) * a.qkv_stride_t;
  for (int d = threadIdx.x; d < D; d += 256) {
    s_q[d] = silu_f(A::ld(row + static_cast<int64_t>(h) * D + d));
    s_k[d] = silu_f(A::ld(row + static_cast<int64_t>(H + h) * D + d));
  }
  float v[4];
  A::ld4(row + 2 * static_cast<int64_t>(H) * D + static_cast<int64_t>(h) * Dv + 4 * c4, v);
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = silu_f(v[e]);
  const float decay = a.decay[h];
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
      const float k = s_k[d], q = s_q[d];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        S[u][e] = fmaf(decay, S[u][e], k * v[e]);
        acc[e] = fmaf(S[u][e], q, acc[e]);
      }
      if (st != nullptr) *reinterpret_cast<f32x4*>(st + static_cast<int64_t>(d) * Dv + 4 * c4) = S[u];
    }
  }
  *reinterpret_cast<f32x4*>(&s_o[threadIdx.x * 4]) = acc;          // [d0][4 c4 + e]
  __syncthreads();
  for (int c = threadIdx.x; c < Dv; c += 256) {
    float o = 0.f;
    for (int g = 0; g < dstep; ++g) o += s_o[(g * Dv4 + c / 4) * 4 + (c & 3)];
    a.out[static_cast<int64_t>(t) * H * Dv + static_cast<int64_t>(h) * Dv + c] = o;
  }
}

inline bool step_shape(const hymeta_lightning_attention_args& a) {
  const int dv4 = a.v_dim / 4;
  const int bytes = a.act_dtype == HYMETA_BF16 ? 2 : 4;
  return a.v_dim % 4 == 0 && dv4 <= 256 && 256 % dv4 == 0 && a.head_dim <= kStepMaxD && reinterpret_cast<uintptr_t>(a.state) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(a.qkv) % (4 * bytes) == 0 && a.qkv_stride_t % 4 == 0 && (2 * a.num_heads * a.head_dim) % 4 == 0;
}

template <typename A>
void launch_rows(const hymeta_lightning_attention_args& a, hipStream_t st, int min_rows, int max_rows) {
  const dim3 grid(a.num_heads, a.num_seqs, (a.v_dim + 255) / 256);
  const dim3 block(a.v_dim >= 256 ? 256 : (a.v_dim + 63) / 64 * 64);
  if (a.head_dim <= 32) hipLaunchKernelGGL((lightning_rows_kernel<A, 32>), grid, block, 0, st, a, min_rows, max_rows);
  else if (a.head_dim <= 64) hipLaunchKernelGGL((lightning_rows_kernel<A, 64>), grid, block, 0, st, a, min_rows, max_rows);
  else if (a.head_dim <= 128) hipLaunchKernelGGL((lightning_rows_kernel<A, 128>), grid, block, 0, st, a, min_rows, max_rows);
  else hipLaunchKernelGGL((lightning_rows_kernel<A, 256>), grid, block, 0, st, a, min_rows, max_rows);
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" size_t hymeta_lightning_attention_workspace_bytes(int32_t num_seqs, int32_t num_heads, int32_t head_dim, int32_t v_dim,
                                                             int32_t max_query_len) {
  if (num_seqs <= 0 || num_heads <= 0 || head_dim <= 0 || v_dim <= 0 || max_query_len < kSegmentMinRows) return 0;
  const size_t nseg = (static_cast<size_t>(max_query_len) + kSegmentRows - 1) / kSegmentRows;
  return nseg * num_seqs * num_heads * head_dim * v_dim * sizeof(float);
}

extern "C" int hymeta_lightning_attention(const hymeta_lightning_attention_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_lightning_attention_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.num_heads <= 0 || a.head_dim <= 0 || a.v_dim <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.head_dim > 256 || a.num_seqs > 65535 || a.v_dim > 256 * 65535) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.qkv || !a.state || !a.decay || !a.out || !a.query_start_loc || !a.context_lens || !a.slot_idx) return HYMETA_ERR_INVALID_ARG;
  if (a.qkv_stride_t < static_cast<int64_t>(a.num_heads) * (2 * a.head_dim + a.v_dim)) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  int max_rows = 0x7fffffff;
  if (chunk_shape(a) && a.max_query_len >= kChunkMinRows) {
    const size_t need = hymeta_lightning_attention_workspace_bytes(a.num_seqs, a.num_heads, a.head_dim, a.v_dim, a.max_query_len);
    const int nseg = need > 0 ? (a.max_query_len + kSegmentRows - 1) / kSegmentRows : 1;
    if (need > 0 && (!a.workspace || a.workspace_bytes < need)) return HYMETA_ERR_WORKSPACE;
    if (static_cast<int64_t>(a.num_seqs) * nseg > 65535) return HYMETA_ERR_UNSUPPORTED;
    const dim3 grid(a.num_heads, a.num_seqs * nseg, a.v_dim / kSliceV);
    auto chunks = [&](int mode) {
      if (a.head_dim == 32) hipLaunchKernelGGL(lightning_chunk_kernel<32>, grid, dim3(256), 0, st, a, kChunkMinRows, kSegmentRows, nseg, mode);
      else if (a.head_dim == 64) hipLaunchKernelGGL(lightning_chunk_kernel<64>, grid, dim3(256), 0, st, a, kChunkMinRows, kSegmentRows, nseg, mode);
      else hipLaunchKernelGGL(lightning_chunk_kernel<128>, grid, dim3(256), 0, st, a, kChunkMinRows, kSegmentRows, nseg, mode);
    };
    if (nseg == 1) {
      chunks(kWhole);
    } else {
      chunks(kSummarise);
      const int64_t per_seq = static_cast<int64_t>(a.num_heads) * a.head_dim * a.v_dim;
      hipLaunchKernelGGL(lightning_chain_kernel, dim3(static_cast<unsigned>((per_seq + 255) / 256), a.num_seqs), dim3(256), 0, st, a, kChunkMinRows,
                         kSegmentRows, nseg);
      chunks(kApply);
    }
    max_rows = kChunkMinRows - 1;
  }
  int min_rows = 1;
  if (step_shape(a)) {
    const dim3 grid(a.num_heads, a.num_seqs);
    if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(lightning_step_kernel<ActBf16>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(lightning_step_kernel<ActF32>, grid, dim3(256), 0, st, a);
    min_rows = 2;
  }
  if (a.max_query_len >= min_rows && max_rows >= min_rows) {
    if (a.act_dtype == HYMETA_BF16) launch_rows<ActBf16>(a, st, min_rows, max_rows);
    else launch_rows<ActF32>(a, st, min_rows, max_rows);
  }
  return launch_status();
}

extern "C" int hymeta_gated_rms_norm(const hymeta_gated_rms_norm_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_gated_rms_norm_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.x || !a.gate || !a.out || a.gate_stride_t < a.width) return HYMETA_ERR_INVALID_ARG;
  const int groups = a.groups > 1 ? a.groups : 1;
  if (a.width % groups != 0 || groups > 65535) return HYMETA_ERR_INVALID_ARG;
  if (a.gate_act != HYMETA_GATE_SIGMOID && a.gate_act != HYMETA_GATE_SILU) return HYMETA_ERR_UNSUPPORTED;
  hipStream_t st = begin_launches(stream);
  if (groups > 1 && a.width / groups <= kGatedWaveCols) {
    const dim3 grid(a.num_tokens, (groups + 3) / 4);
    if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(gated_rms_norm_wave_kernel<ActBf16>, grid, dim3(256), 0, st, a, groups);
    else hipLaunchKernelGGL(gated_rms_norm_wave_kernel<ActF32>, grid, dim3(256), 0, st, a, groups);
    return launch_status();
  }
  const bool cached = a.width / groups <= kGatedCached;
  if (a.act_dtype == HYMETA_BF16) {
    if (cached) hipLaunchKernelGGL((gated_rms_norm_kernel<ActBf16, true>), dim3(a.num_tokens, groups), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((gated_rms_norm_kernel<ActBf16, false>), dim3(a.num_tokens, groups), dim3(256), 0, st, a);
  } else {
    if (cached) hipLaunchKernelGGL((gated_rms_norm_kernel<ActF32, true>), dim3(a.num_tokens, groups), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((gated_rms_norm_kernel<ActF32, false>), dim3(a.num_tokens, groups), dim3(256), 0, st, a);
  }
  return launch_status();
}
