// Causal paged attention with a distance bias and a sink, for any head size, fp32 or bf16 rows:
// the per-head query / key norm with the paged key / value write, and the attention itself.
//
// Scores, the running maximum, the weights and the weighted sum of the values are fp32 whatever the
// activation type.  The sink is a key of score 0 without a value: the running maximum starts at 0
// and the denominator at exp(0 - 0) = 1, everything else is the ordinary streaming softmax.
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kMaxHeadDim = 4096;
constexpr int kMaxVChunks = 8;       // value size <= 512

// grid = tokens; a wave per (token, head) task: query heads, then key heads, then value heads.
template <typename A>
__global__ __launch_bounds__(256) void qk_norm_cache_kernel(hymeta_qk_norm_cache_args a) {
  typedef typename A::elem elem;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int H = a.num_heads, G = a.num_kv_heads, D = a.head_dim, Dv = a.v_dim;
  elem* row = static_cast<elem*>(a.qkv) + t * a.qkv_stride_t;
  const int64_t slot = a.slot_mapping ? a.slot_mapping[t] : -1;
  const bool store = slot >= 0 && slot < a.num_blocks * a.block_size;
  elem* cache = static_cast<elem*>(a.kv_cache) + (store ? slot : 0) * G * static_cast<int64_t>(D + Dv);
  for (int task = wave; task < H + 2 * G; task += 4) {
    if (task < H + G) {
      const bool is_q = task < H;
      elem* src = row + static_cast<int64_t>(task) * D;          // q heads, then k heads, contiguous
      const float* w = is_q ? a.q_weight : a.k_weight;
      if (!is_q && !store && w == nullptr) continue;
      float inv = 1.f;
      if (w != nullptr) {
        float ss = 0.f;
        for (int d = lane; d < D; d += 64) {
          const float v = A::ld(src + d);
          ss += v * v;
        }
        ss = wave_sum(ss);
        inv = 1.f / sqrtf(ss / static_cast<float>(D) + a.eps);
      }
      elem* dst = is_q ? src : cache + static_cast<int64_t>(task - H) * (D + Dv);
      if (is_q && w == nullptr) continue;
      if (!is_q && !store) continue;
      for (int d = lane; d < D; d += 64) {
        const float v = A::ld(src + d);
        A::st(dst + d, w ? v * inv * w[d] : v);
      }
    } else if (store) {
      const int g = task - H - G;
      const elem* src = row + static_cast<int64_t>(H + G) * D + static_cast<int64_t>(g) * Dv;
      elem* dst = cache + static_cast<int64_t>(g) * (D + Dv) + D;
      for (int d = lane; d < Dv; d += 64) dst[d] = src[d];
    }
  }
}

__device__ __forceinline__ float distance_bias(int mode, float a, float b, int dist) {
  return mode == HYMETA_BIAS_LOG_DISTANCE ? a * log1pf(b * static_cast<float>(dist)) : 0.f;
}

// One wave per (query row, head).  Keys in tiles of 64: lane = key for the scores, lane = value channel for the
// weighted sum, the tile's weights and row addresses handed over through LDS.
template <typename A>
__global__ __launch_bounds__(64) void sink_attention_rows_kernel(hymeta_sink_attention_args a) {
  typedef typename A::elem elem;
  __shared__ float s_q[kMaxHeadDim];
  __shared__ float s_p[64];
  __shared__ int64_t s_row[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int D = a.head_dim, Dv = a.v_dim, G = a.num_kv_heads;
  const int g = h / (a.num_heads / G);
  const int s = seq_of_row(a.query_start_loc, a.num_seqs, t);
  const int pos = a.seq_lens[s] - (a.query_start_loc[s + 1] - t);
  if (pos < 0) return;
  const int first = a.window_left >= 0 ? max(0, pos - a.window_left) : 0;
  const elem* q = static_cast<const elem*>(a.q) + static_cast<int64_t>(t) * a.q_stride_t + static_cast<int64_t>(h) * D;
  for (int d = lane; d < D; d += 64) s_q[d] = A::ld(q + d);
  const int32_t* bt = a.block_tables + static_cast<int64_t>(s) * a.block_table_stride;
  const elem* cache = static_cast<const elem*>(a.kv_cache);
  // where the head's key and value lie in a cache row: a key followed by its value per key/value head; a key whose first Dv
  // elements are the value; or one key for all heads followed by the key/value heads' values
  int64_t row_elems, key_off, val_off;
  if (a.kv_layout == HYMETA_KV_SHARED_KEY) row_elems = D + static_cast<int64_t>(G) * Dv, key_off = 0, val_off = D + static_cast<int64_t>(g) * Dv;
  else if (a.kv_layout == HYMETA_KV_VALUE_IN_KEY) row_elems = static_cast<int64_t>(G) * D, key_off = static_cast<int64_t>(g) * D, val_off = key_off;
  else row_elems = static_cast<int64_t>(G) * (D + Dv), key_off = static_cast<int64_t>(g) * (D + Dv), val_off = key_off + D;
  const float ba = a.bias_mode ? a.bias_a[h] : 0.f, bb = a.bias_mode ? a.bias_b[h] : 0.f;
  // the sink: a key of score sink_logits[h] (0 without) that has no value
  float m = a.sink ? (a.sink_logits ? a.sink_logits[h] : 0.f) : -INFINITY, l = a.sink ? 1.f : 0.f;
  float acc[kMaxVChunks] = {};
  const int nvc = (Dv + 63) / 64;
  __syncthreads();
  // two runs of keys: the kept first ones that lie before the window, then the window
  const int kept = a.window_left >= 0 ? min(a.keep_first, first) : 0;
  for (int run = 0; run < 2; ++run) {
    const int lo = run == 0 ? 0 : first, hi = run == 0 ? kept - 1 : pos;
    for (int j0 = lo; j0 <= hi; j0 += 64) {
      const int j = j0 + lane;
      const bool valid = j <= hi;
      float sc = -INFINITY;
      int64_t roff = 0;
      if (valid) {
        const int64_t blk = bt[j / a.block_size];
        roff = (blk * a.block_size + j % a.block_size) * row_elems;
        const elem* k = cache + roff + key_off;
        float dot = 0.f;
        for (int d = 0; d < D; ++d) dot = fmaf(s_q[d], A::ld(k + d), dot);
        sc = dot * a.scale;
        if (a.softcap > 0.f) sc = a.softcap * tanhf(sc / a.softcap);
        sc -= distance_bias(a.bias_mode, ba, bb, pos - j);
      }
      const float m_new = fmaxf(m, wave_max(sc));
      const float p = valid ? expf(sc - m_new) : 0.f;
      const float corr = expf(m - m_new);            // m = -inf only without a sink before the first tile: corr = 0, l = 0
      l = l * corr + wave_sum(p);
      m = m_new;
      __syncthreads();
      s_p[lane] = p;
      s_row[lane] = roff + val_off;
      __syncthreads();
      const int n = min(64, hi - j0 + 1);
#pragma unroll
      for (int cc = 0; cc < kMaxVChunks; ++cc) {
        if (cc < nvc) {
          const int c = cc * 64 + lane;
          float r = acc[cc] * corr;
          if (c < Dv)
            for (int jj = 0; jj < n; ++jj) r = fmaf(s_p[jj], A::ld(cache + s_row[jj] + c), r);
          acc[cc] = r;
        }
      }
    }
  }
  elem* out = static_cast<elem*>(a.out) + (static_cast<int64_t>(t) * a.num_heads + h) * Dv;
  float inv = l > 0.f ? 1.f / l : 0.f;
  if (a.head_gate) inv *= sigmoid_exact(A::ld(static_cast<const elem*>(a.head_gate) + static_cast<int64_t>(t) * a.head_gate_stride_t + h));
#pragma unroll
  for (int cc = 0; cc < kMaxVChunks; ++cc) {
    const int c = cc * 64 + lane;
    if (cc < nvc && c < Dv) A::st(out + c, acc[cc] * inv);
  }
}


// ------------------------------------------------------------------------------------------------
// bf16 on the matrix cores.  A wave owns 32 "rows" (two blocks of 16): in a prompt's portion 32 consecutive query
// rows of one head, in a decode step the query heads of one key/value head (they share every key and value row they
// read).  Keys come in tiles of 64 through LDS: the key rows as they lie in the pages, the value rows transposed, so
// that both are read as MFMA operands with 8- and 16-byte LDS loads.
//
//   S^T[key][row] = K[key][:] . Q[row][:]           v_mfma_f32_16x16x32_bf16, A = K fragment, B = Q fragment
//   O^T[c][row]  += V^T[c][key] P^T[key][row]       A = V^T fragment, B = P^T
//
// The transposed forms make the result layout of the first product (a lane holds 4 consecutive keys of one row) the
// B-operand layout of the second, so the weights never leave their registers, and they leave the row statistics in the
// lane that owns the row in both products.  The weights stay fp32-exact through the bf16 matrix product: p = hi + lo
// with hi = bf16(p), lo = bf16(p - hi), two products (relative error of p 2^-17 instead of 2^-9).
// ------------------------------------------------------------------------------------------------
typedef float f32x4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4v mfma16(bf16x8 a, bf16x8 b, f32x4v c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Row blocks of 16 a prompt's wave holds.  Two halve the LDS reads per matrix instruction, but at about 250 registers
// leave one workgroup per compute unit: measured on prompts of 2048 / 4096 / 8192 rows (28 heads of 128) 0.20 / 0.59 /
// 2.10 ms against 0.21 / 0.64 / 1.86 ms with one.
#ifndef PREFILL_RB
#define PREFILL_RB 1
#endif
constexpr int kTileKeys = 64;
constexpr int kRowsPerWave = 32;

// The value columns one launch computes: `first` .. `first` + DV of the `total` columns of a value row (and of an output
// row).  Values wider than the kernels' DV run as several launches over slices (each repeats the scores).
struct ValueSlice {
  int first, total;
  // (decode form) the query heads of a key/value head one launch takes as its rows: h_first .. h_first + h_count of the
  // group; h_count 0: the whole group.  Groups of more than 32 heads run as several launches.
  int h_first = 0, h_count = 0;
};

template <int D, int DV>
struct MfmaSmem {
  static constexpr int kPitchK = D + 8;               // bf16 elements per key row (16-byte reads of 16 rows: no bank conflict)
  static constexpr int kPitchV = kTileKeys + 8;       // bf16 elements per value channel
  uint16_t k[kTileKeys * kPitchK];
  uint16_t vt[DV * kPitchV];
};

// Staging of keys [j0, j0 + 64) of a sequence's key/value head g, in two halves so that the loads of the next tile
// are in flight while the current one is multiplied: `issue` reads 16-byte chunks into registers (keys past `last` read
// as zero), `commit` stores them into LDS.  A key row goes in as it is.  The value rows go in transposed: a thread takes
// the same 8 channels of 4 consecutive keys (4 chunks), which are 8 runs of 4 keys in the transposed image, one 8-byte
// store each.  The 4-key groups of a channel are permuted by the channel's chunk number (XOR), which spreads the stores
// of threads that hold the same keys over the banks; the reader applies the same permutation.
// Layout (enum hymeta_kv_layout).  VALUE_IN_KEY: a head's part of a cache row is its key alone (D elements), whose first DV
// elements are also its value.  SHARED_KEY: a row is one key of D elements for all heads, then num_kv_heads values of DV.
template <int D, int DV, int Threads, int Layout>
struct TileStage {
  static constexpr bool VinK = Layout == HYMETA_KV_VALUE_IN_KEY, Shared = Layout == HYMETA_KV_SHARED_KEY;
  static constexpr int kKeyChunksPerRow = D / 8, kValChunksPerRow = DV / 8;
  static constexpr int kKeyChunks = kTileKeys * kKeyChunksPerRow;
  static constexpr int kKeyPerThread = (kKeyChunks + Threads - 1) / Threads;
  static constexpr int kValBlocks = (kTileKeys / 4) * kValChunksPerRow;       // (4 keys) x (8 channels) each
  static constexpr int kHeadElems = VinK ? D : D + DV, kValueAt = VinK ? 0 : D;
  static_assert(D % 32 == 0 && DV % 16 == 0 && kValBlocks <= Threads && (!VinK || DV <= D), "the staging roles fit the workgroup");
  u32x4 rk[kKeyPerThread];
  u32x4 rv[4];
  int value_at = kValueAt;      // where the staged value columns start in a head's part of a row

  // Pages hold a power of two of rows here (the host sends other sizes to the plain kernel).  A page of 64 rows or more
  // holds a whole tile (tiles start at multiples of 64): its number is one scalar load per tile, not a dependent vector
  // load in front of every row's loads.
  struct Pages {
    const uint16_t* cache;
    const int32_t* bt;
    int64_t row_elems, head_off;
    int shift, mask;
    int64_t tile_base;          // first row of the tile's page, in rows of the cache (pages of >= 64 rows)
    bool whole;
  };

  static __device__ __forceinline__ Pages pages(const hymeta_sink_attention_args& a, const int32_t* bt, int g, int j0) {
    Pages p;
    p.cache = static_cast<const uint16_t*>(a.kv_cache);
    p.bt = bt;
    p.row_elems = Shared ? D + static_cast<int64_t>(a.num_kv_heads) * DV : static_cast<int64_t>(a.num_kv_heads) * kHeadElems;
    p.head_off = Shared ? 0 : static_cast<int64_t>(g) * kHeadElems;
    p.shift = __builtin_ctz(a.block_size);
    p.mask = a.block_size - 1;
    p.whole = a.block_size >= kTileKeys;
    p.tile_base = 0;
    if (p.whole) p.tile_base = (static_cast<int64_t>(__builtin_amdgcn_readfirstlane(bt[j0 >> p.shift])) << p.shift) + (j0 & p.mask);
    return p;
  }

  static __device__ __forceinline__ const uint16_t* row_ptr(const Pages& p, int j0, int j) {
    const int64_t row = p.whole ? p.tile_base + (j - j0) : (static_cast<int64_t>(p.bt[j >> p.shift]) << p.shift) + (j & p.mask);
    return p.cache + row * p.row_elems + p.head_off;
  }

  __device__ __forceinline__ void issue(const hymeta_sink_attention_args& a, const int32_t* bt, int g, int j0, int last) {
    const Pages p = pages(a, bt, g, j0);
#pragma unroll
    for (int i = 0; i < kKeyPerThread; ++i) {
      const int idx = i * Threads + threadIdx.x;
      const int j = j0 + idx / kKeyChunksPerRow;
      rk[i] = u32x4{0u, 0u, 0u, 0u};
      if (j <= last && (kKeyChunks % Threads == 0 || idx < kKeyChunks)) rk[i] = ld16g(row_ptr(p, j0, j) + (idx % kKeyChunksPerRow) * 8);
    }
    if (static_cast<int>(threadIdx.x) < kValBlocks) {
      const int ch = threadIdx.x % kValChunksPerRow, grp = threadIdx.x / kValChunksPerRow;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = j0 + 4 * grp + i;
        rv[i] = u32x4{0u, 0u, 0u, 0u};
        if (j <= last) rv[i] = ld16g(row_ptr(p, j0, j) + value_at + ch * 8);
      }
    }
  }

  __device__ __forceinline__ void commit(MfmaSmem<D, DV>& sm) const {
#pragma unroll
    for (int i = 0; i < kKeyPerThread; ++i) {
      const int idx = i * Threads + threadIdx.x;
      if (kKeyChunks % Threads == 0 || idx < kKeyChunks)
        st16(&sm.k[(idx / kKeyChunksPerRow) * MfmaSmem<D, DV>::kPitchK + (idx % kKeyChunksPerRow) * 8], rk[i]);
    }
    if (static_cast<int>(threadIdx.x) < kValBlocks) {
      const int ch = threadIdx.x % kValChunksPerRow, grp = threadIdx.x / kValChunksPerRow;
      uint16_t* dst = &sm.vt[(8 * ch) * MfmaSmem<D, DV>::kPitchV + 4 * (grp ^ (ch & 15))];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int dw = e >> 1;
        u32x2 v;
        if (e & 1) {
          v[0] = (rv[0][dw] >> 16) | (rv[1][dw] & 0xffff0000u);
          v[1] = (rv[2][dw] >> 16) | (rv[3][dw] & 0xffff0000u);
        } else {
          v[0] = (rv[0][dw] & 0xffffu) | (rv[1][dw] << 16);
          v[1] = (rv[2][dw] & 0xffffu) | (rv[3][dw] << 16);
        }
        *reinterpret_cast<u32x2*>(dst + e * MfmaSmem<D, DV>::kPitchV) = v;
      }
    }
  }
};

// Where the 4-key group `grp` (0 .. 15) of value channel c lies in the transposed image.
template <int D, int DV>
__device__ __forceinline__ const uint16_t* vt_group(const MfmaSmem<D, DV>& sm, int c, int grp) {
  return &sm.vt[c * MfmaSmem<D, DV>::kPitchV + 4 * (grp ^ ((c >> 3) & 15))];
}

// The rows of one wave against the staged tile.  RB row blocks of 16 (row = 16 rb + lane % 16); the wave takes NKS of the
// tile's four 16-key subtiles, from ks_lo on (a prompt's wave all four, a decode wave one: the four waves of a decode
// workgroup split every tile between them and each keeps statistics of its own).
template <int D, int DV, int RB>
struct WaveRows {
  bf16x8 q[RB][D / 32];
  f32x4v o[RB][DV / 16];
  float m[RB], l[RB];          // running maximum of the row; this lane's share of the denominator
  int pos[RB];                 // position of the row's query (-1: no such row)
  float ba[RB], bb[RB];
};

typedef short bf16x4 __attribute__((ext_vector_type(4)));

// tanh through the hardware's exponential: 1 - 2 / (exp(2 x) + 1), exact at both ends (exp2 -> inf gives 1, -> 0 gives -1)
__device__ __forceinline__ float tanh_fast(float x) {
  return 1.f - 2.f * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(x * 2.8853900817779268f) + 1.f);
}

template <int D, int DV, int RB, int NKS, bool Masked>
__device__ __forceinline__ void attend_tile(WaveRows<D, DV, RB>& w, const MfmaSmem<D, DV>& sm, const hymeta_sink_attention_args& a,
                                            int j0, int ks_lo) {
  static_assert(NKS == 4 || NKS == 1, "all of a tile's subtiles or one");
  const int lane = threadIdx.x & 63, n = lane & 15, g4 = lane >> 4;
  constexpr int PK = MfmaSmem<D, DV>::kPitchK;
  f32x4v s[RB][NKS];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) s[rb][ks] = f32x4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
    for (int st = 0; st < D / 32; ++st) {
      const bf16x8 kf = __builtin_bit_cast(bf16x8, ld16(&sm.k[(16 * (ks_lo + ks) + n) * PK + 32 * st + 8 * g4]));
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) s[rb][ks] = mfma16(kf, w.q[rb][st], s[rb][ks]);
    }
  // lane holds, per row block, the scores of its row (n) against keys j0 + 16 (ks_lo + ks) + 4 g4 + r.  Everything from
  // here to the weights is in the base-2 domain (scores times log2 e; the bias' coefficient is unchanged, as
  // a ln x * log2 e = a log2 x): one v_log and one v_exp per score and no multiplications around them.  The running
  // maximum, and with it the sink's score 0, mean the same in both domains.
  const float scale2 = a.scale * 1.4426950408889634f;
  const bool bias = a.bias_mode == HYMETA_BIAS_LOG_DISTANCE;
  // capped scores: softcap tanh(score / softcap), moved into the base-2 domain like the others
  const bool capped = a.softcap > 0.f;
  const float cap2 = a.softcap * 1.4426950408889634f, cap_in = capped ? a.scale / a.softcap : 0.f;
  uint32_t phi[RB][NKS][2], plo[RB][NKS][2];       // the weights' bf16 high and low parts, two per dword
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int pos = w.pos[rb];
    // distance of the lane's key r of subtile ks: fd0 - (16 ks + r)
    const float fd0 = static_cast<float>(pos - j0 - 16 * ks_lo - 4 * g4);
    float mx = -INFINITY;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float sc = s[rb][ks][r] * scale2;
        if (capped) sc = cap2 * tanh_fast(s[rb][ks][r] * cap_in);
        if (bias) sc = fmaf(-w.ba[rb], __log2f(fmaf(w.bb[rb], fd0 - static_cast<float>(16 * ks + r), 1.f)), sc);
        if (Masked) {
          const int j = j0 + 16 * (ks_lo + ks) + 4 * g4 + r;
          const int first = a.window_left >= 0 ? pos - a.window_left : 0;
          sc = (j <= pos && (j >= first || j < a.keep_first)) ? sc : -INFINITY;
        }
        s[rb][ks][r] = sc;
        mx = fmaxf(mx, sc);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(w.m[rb], mx);
    // (masked tiles only) a row with nothing visible so far and no sink keeps m = -inf: weights and correction are 0
    const bool empty = Masked && m_new == -INFINITY;
    const float corr = empty ? 0.f : __builtin_amdgcn_exp2f(w.m[rb] - m_new);
    float sum = 0.f;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
      for (int r2 = 0; r2 < 2; ++r2) {
        float p[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          p[u] = empty ? 0.f : __builtin_amdgcn_exp2f(s[rb][ks][2 * r2 + u] - m_new);
          sum += p[u];
        }
        const uint32_t hi = pack_bf16x2(p[0], p[1]);
        phi[rb][ks][r2] = hi;
        plo[rb][ks][r2] = pack_bf16x2(p[0] - lo_bf(hi), p[1] - hi_bf(hi));
      }
    w.l[rb] = w.l[rb] * corr + sum;
    w.m[rb] = m_new;
#pragma unroll
    for (int cb = 0; cb < DV / 16; ++cb) w.o[rb][cb] *= corr;
  }
  if constexpr (NKS == 4) {
#pragma unroll
    for (int cb = 0; cb < DV / 16; ++cb)
#pragma unroll
      for (int kp = 0; kp < 2; ++kp) {
        // k index 8 g4 + e of the product: keys 16 (2 kp) + 4 g4 + e for e < 4, 16 (2 kp + 1) + 4 g4 + e - 4 after
        const u32x2 v0 = *reinterpret_cast<const u32x2*>(vt_group<D, DV>(sm, 16 * cb + n, 8 * kp + g4));
        const u32x2 v1 = *reinterpret_cast<const u32x2*>(vt_group<D, DV>(sm, 16 * cb + n, 8 * kp + 4 + g4));
        const bf16x8 vf = __builtin_bit_cast(bf16x8, (u32x4{v0[0], v0[1], v1[0], v1[1]}));
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const bf16x8 ph = __builtin_bit_cast(bf16x8, (u32x4{phi[rb][2 * kp][0], phi[rb][2 * kp][1], phi[rb][2 * kp + 1][0], phi[rb][2 * kp + 1][1]}));
          const bf16x8 pl = __builtin_bit_cast(bf16x8, (u32x4{plo[rb][2 * kp][0], plo[rb][2 * kp][1], plo[rb][2 * kp + 1][0], plo[rb][2 * kp + 1][1]}));
          w.o[rb][cb] = mfma16(vf, ph, w.o[rb][cb]);
          w.o[rb][cb] = mfma16(vf, pl, w.o[rb][cb]);
        }
      }
  } else {
#pragma unroll
    for (int cb = 0; cb < DV / 16; ++cb) {
      const bf16x4 vf = __builtin_bit_cast(bf16x4, *reinterpret_cast<const u32x2*>(vt_group<D, DV>(sm, 16 * cb + n, 4 * ks_lo + g4)));
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const bf16x4 ph = __builtin_bit_cast(bf16x4, (u32x2{phi[rb][0][0], phi[rb][0][1]}));
        const bf16x4 pl = __builtin_bit_cast(bf16x4, (u32x2{plo[rb][0][0], plo[rb][0][1]}));
        w.o[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, ph, w.o[rb][cb], 0, 0, 0);
        w.o[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pl, w.o[rb][cb], 0, 0, 0);
      }
    }
  }
}

template <int D, int DV, int RB>
__device__ __forceinline__ void load_q(WaveRows<D, DV, RB>& w, int rb, const uint16_t* qrow) {
  const int g4 = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int st = 0; st < D / 32; ++st)
    w.q[rb][st] = qrow ? __builtin_bit_cast(bf16x8, ld16g(qrow + 32 * st + 8 * g4)) : bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
}

// Waves of a prompt workgroup: 8, or 4 for keys longer than 192 elements, whose query fragments (D / 8 registers) and
// staging registers do not leave a wave of 8 its accumulators within 256 registers (408 bytes of scratch per lane at
// 576; a workgroup of 4 waves has 512 registers per wave).
template <int D> struct PrefillWaves { static constexpr int value = D > 192 ? 4 : 8; };
template <int RB, int Waves> struct PrefillShape { static constexpr int kRows = 16 * RB * Waves; };

// Portions of prompts: grid = (tiles of 16 RB rows per wave, heads, sequences); a wave holds RB blocks of 16 rows; sequences with
// one row are left to the decode form.
template <int D, int DV, int RB, int Layout>
__global__ __launch_bounds__(64 * PrefillWaves<D>::value) void sink_attention_prefill_mfma_kernel(hymeta_sink_attention_args a, ValueSlice vs) {
  constexpr int kPrefillWaves = PrefillWaves<D>::value;
  constexpr int kRows = PrefillShape<RB, kPrefillWaves>::kRows;
  constexpr int kImages = 2 * sizeof(MfmaSmem<D, DV>) <= 159 * 1024 ? 2 : 1;        // (160 KB of LDS)
  __shared__ MfmaSmem<D, DV> sm[kImages];
  const int s = blockIdx.z, h = blockIdx.y;
  const int row0 = a.query_start_loc[s];
  const int q = a.query_start_loc[s + 1] - row0;
  if (q <= 1 || static_cast<int>(blockIdx.x) * kRows >= q) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 15, g4 = lane >> 4;
  const int g = h / (a.num_heads / a.num_kv_heads);
  const int ctx = a.seq_lens[s] - q;
  const int32_t* bt = a.block_tables + static_cast<int64_t>(s) * a.block_table_stride;
  WaveRows<D, DV, RB> w;
  const int wrow = blockIdx.x * kRows + wave * 16 * RB;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int r = wrow + 16 * rb + n;
    const bool ok = r < q;
    w.pos[rb] = ok ? ctx + r : -1;
    w.ba[rb] = a.bias_mode ? a.bias_a[h] : 0.f;
    w.bb[rb] = a.bias_mode ? a.bias_b[h] : 0.f;
    w.m[rb] = a.sink ? (a.sink_logits ? a.sink_logits[h] * 1.4426950408889634f : 0.f) : -INFINITY;
    w.l[rb] = (a.sink && g4 == 0) ? 1.f : 0.f;        // the sink's exp(m - m), counted once per row
    load_q<D, DV, RB>(w, rb, ok ? static_cast<const uint16_t*>(a.q) + static_cast<int64_t>(row0 + r) * a.q_stride_t + static_cast<int64_t>(h) * D : nullptr);
#pragma unroll
    for (int cb = 0; cb < DV / 16; ++cb) w.o[rb][cb] = f32x4v{0.f, 0.f, 0.f, 0.f};
  }
  const int block_last = ctx + min(q, static_cast<int>(blockIdx.x) * kRows + kRows) - 1;      // last key any row of the block sees
  const int wave_last = ctx + min(q, wrow + 16 * RB) - 1;
  int j_first = 0;
  if (a.window_left >= 0) j_first = max(0, ctx + static_cast<int>(blockIdx.x) * kRows - a.window_left) / kTileKeys * kTileKeys;
  // the tiles of the kept first keys that lie before the window's first tile come first, then the window's
  const int keep_end = a.window_left >= 0 ? min((a.keep_first + kTileKeys - 1) / kTileKeys * kTileKeys, j_first) : 0;
  const int j_start = keep_end > 0 ? 0 : j_first;
  auto next = [&](int j0) { return (j0 < keep_end && j0 + kTileKeys >= keep_end) ? j_first : j0 + kTileKeys; };
  // two LDS images: while the waves multiply tile t out of one, tile t + 1 goes into the other and the loads of tile
  // t + 2 are in flight; one barrier per tile
  TileStage<D, DV, 64 * kPrefillWaves, Layout> stage;
  if (Layout == HYMETA_KV_VALUE_IN_KEY) stage.value_at = vs.first;
  if (Layout == HYMETA_KV_SHARED_KEY) stage.value_at = D + g * DV;
  stage.issue(a, bt, g, j_start, block_last);
  stage.commit(sm[0]);
  if (kImages == 2 && next(j_start) <= block_last) stage.issue(a, bt, g, next(j_start), block_last);
  __syncthreads();
  if constexpr (kImages == 2) {
    int buf = 0;
    for (int j0 = j_start; j0 <= block_last; j0 = next(j0), buf ^= 1) {
      const int j1 = next(j0), j2 = next(j1);
      if (j1 <= block_last) stage.commit(sm[buf ^ 1]);
      if (j2 <= block_last) stage.issue(a, bt, g, j2, block_last);
      if (wrow < q && j0 <= wave_last) {
        // tiles wholly before the wave's first row (and no window) need no mask: every key is visible to every row
        if (a.window_left < 0 && j0 + kTileKeys - 1 <= ctx + wrow) attend_tile<D, DV, RB, 4, false>(w, sm[buf], a, j0, 0);
        else attend_tile<D, DV, RB, 4, true>(w, sm[buf], a, j0, 0);
      }
      __syncthreads();
    }
  } else {
    // one image (tiles of long rows): the next tile's loads are in flight while this one is multiplied and go into LDS
    // behind a barrier
    for (int j0 = j_start; j0 <= block_last; j0 = next(j0)) {
      const bool more = next(j0) <= block_last;
      if (more) stage.issue(a, bt, g, next(j0), block_last);
      if (wrow < q && j0 <= wave_last) {
        if (a.window_left < 0 && j0 + kTileKeys - 1 <= ctx + wrow) attend_tile<D, DV, RB, 4, false>(w, sm[0], a, j0, 0);
        else attend_tile<D, DV, RB, 4, true>(w, sm[0], a, j0, 0);
      }
      __syncthreads();
      if (more) {
        stage.commit(sm[0]);
        __syncthreads();
      }
    }
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float l = w.l[rb];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    const int r = wrow + 16 * rb + n;
    if (r >= q) continue;
    float inv = l > 0.f ? 1.f / l : 0.f;
    if (a.head_gate) inv *= sigmoid_exact(bf2f(static_cast<const uint16_t*>(a.head_gate)[static_cast<int64_t>(row0 + r) * a.head_gate_stride_t + h]));
    uint16_t* out = static_cast<uint16_t*>(a.out) + (static_cast<int64_t>(row0 + r) * a.num_heads + h) * vs.total + vs.first;
#pragma unroll
    for (int cb = 0; cb < DV / 16; ++cb) {
      const f32x4v o = w.o[rb][cb] * inv;
      *reinterpret_cast<u32x2*>(out + 16 * cb + 4 * g4) = u32x2{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
    }
  }
}

// Partial of a (sequence, key/value head, slice, wave): per query head of the group DV weighted values, then the
// maximum and denominator, rows padded to whole 16 bytes.
__host__ __device__ inline size_t partial_row_floats(int dv) { return static_cast<size_t>(dv) + 4; }
constexpr int kDecodeWaves = 4;
// LDS images of a decode workgroup: two (the next tile goes into the other image while this one is multiplied) where
// both fit in 72 KB, which leaves two workgroups on a compute unit; one for larger tiles, so that three or four
// workgroups overlap each other instead.
template <int D, int DV>
struct DecodeImages {
  static constexpr int value = 2 * sizeof(MfmaSmem<D, DV>) <= 72 * 1024 ? 2 : 1;
};
// Whether the four waves of a decode workgroup merge their partials through LDS (the tile images, free after the last
// tile, hold two waves' rows at a time: waves 2, 3 hand theirs to waves 0, 1, then wave 1 to wave 0) and write one
// partial per slice: a quarter of the partials' traffic and of the combine's work.
template <int D, int DV, int RB>
struct DecodeMerge {
  static constexpr bool value = DecodeImages<D, DV>::value * sizeof(MfmaSmem<D, DV>) >= sizeof(float) * 2 * 16 * RB * (DV + 4);
};

// Decode: a workgroup per (sequence with one row, key/value head, slice of the keys); rows = the group's query heads; the
// four waves share the staged tiles and take a 16-key subtile each.  Every wave writes its (maximum, denominator,
// weighted values) per head; the combine kernel merges them and the sink.
template <int D, int DV, int RB, int Layout>
__global__ __launch_bounds__(64 * kDecodeWaves) void sink_attention_decode_mfma_kernel(hymeta_sink_attention_args a, int splits, int tiles_per_split, ValueSlice vs) {
  constexpr int kImages = DecodeImages<D, DV>::value;
  __shared__ MfmaSmem<D, DV> sm[kImages];
  int s = blockIdx.z, g = blockIdx.y, split = blockIdx.x;
  if (Layout == HYMETA_KV_SHARED_KEY) {
    // The value groups of a (sequence, split) read the same key tiles.  Workgroups go to the chip's 8 dies (each with an
    // L2 of its own) round robin by their number: a one-dimensional grid numbered so that those groups follow each other
    // on ONE die, which then fetches the keys from memory once instead of once per group.
    const int chunk = blockIdx.x >> 3, die = blockIdx.x & 7;
    const int pair = (chunk / a.num_kv_heads) * 8 + die;
    if (pair >= splits * a.num_seqs) return;
    g = chunk % a.num_kv_heads, s = pair / splits, split = pair % splits;
  }
  const int t = a.query_start_loc[s];
  if (a.query_start_loc[s + 1] - t != 1) return;
  const int pos = a.seq_lens[s] - 1;
  const int group = a.num_heads / a.num_kv_heads;
  const int HG = vs.h_count ? vs.h_count : group;            // this launch's rows
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 15, g4 = lane >> 4;
  // The sequence's tiles, numbered v = 0 ..: without a window tile v holds the keys from 64 v on, split as the host says.
  // With a window: the tiles of the kept first keys that lie before the window's first tile, then the window's tiles
  // (tiles wholly before the window are not read), dealt evenly over the splits.
  int kept_tiles = 0, window_from = 0, num_tiles = pos / kTileKeys + 1, per = tiles_per_split;
  if (a.window_left >= 0) {
    window_from = max(0, pos - a.window_left) / kTileKeys * kTileKeys;
    kept_tiles = min((a.keep_first + kTileKeys - 1) / kTileKeys * kTileKeys, window_from) / kTileKeys;
    num_tiles = kept_tiles + (pos - window_from) / kTileKeys + 1;
    per = (num_tiles + splits - 1) / splits;
  }
  const int v_lo = split * per, v_hi = min(num_tiles, v_lo + per) - 1;
  auto tile = [&](int v) { return v < kept_tiles ? v * kTileKeys : window_from + (v - kept_tiles) * kTileKeys; };
  constexpr bool kMerge = DecodeMerge<D, DV, RB>::value;
  float* part = static_cast<float*>(a.workspace) +
                (((static_cast<size_t>(s) * a.num_kv_heads + g) * splits + split) * (kMerge ? 1 : kDecodeWaves) + (kMerge ? 0 : wave)) *
                    (HG * partial_row_floats(DV));
  const int32_t* bt = a.block_tables + static_cast<int64_t>(s) * a.block_table_stride;
  WaveRows<D, DV, RB> w;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int r = 16 * rb + n;
    const bool ok = r < HG;
    const int h = g * group + vs.h_first + (ok ? r : 0);
    w.pos[rb] = ok ? pos : -1;
    w.ba[rb] = a.bias_mode ? a.bias_a[h] : 0.f;
    w.bb[rb] = a.bias_mode ? a.bias_b[h] : 0.f;
    w.m[rb] = -INFINITY;
    w.l[rb] = 0.f;
    load_q<D, DV, RB>(w, rb, ok ? static_cast<const uint16_t*>(a.q) + static_cast<int64_t>(t) * a.q_stride_t + static_cast<int64_t>(h) * D : nullptr);
#pragma unroll
    for (int cb = 0; cb < DV / 16; ++cb) w.o[rb][cb] = f32x4v{0.f, 0.f, 0.f, 0.f};
  }
  TileStage<D, DV, 64 * kDecodeWaves, Layout> stage;
  if (Layout == HYMETA_KV_VALUE_IN_KEY) stage.value_at = vs.first;
  if (Layout == HYMETA_KV_SHARED_KEY) stage.value_at = D + g * DV;
  if (v_lo <= v_hi) {
    stage.issue(a, bt, g, tile(v_lo), pos);
    stage.commit(sm[0]);
    if (kImages == 2 && v_lo + 1 <= v_hi) stage.issue(a, bt, g, tile(v_lo + 1), pos);
  }
  __syncthreads();
  if constexpr (kImages == 2) {
    int buf = 0;
    for (int v = v_lo; v <= v_hi; ++v, buf ^= 1) {
      const int j0 = tile(v);
      if (v + 1 <= v_hi) stage.commit(sm[buf ^ 1]);
      if (v + 2 <= v_hi) stage.issue(a, bt, g, tile(v + 2), pos);
      if (j0 + 16 * wave <= pos) {
        if (a.window_left < 0 && j0 + kTileKeys - 1 <= pos) attend_tile<D, DV, RB, 1, false>(w, sm[buf], a, j0, wave);
        else attend_tile<D, DV, RB, 1, true>(w, sm[buf], a, j0, wave);
      }
      __syncthreads();
    }
  } else {
    // one image: the next tile's loads are in flight while this one is multiplied and go into LDS behind a barrier
    for (int v = v_lo; v <= v_hi; ++v) {
      const int j0 = tile(v);
      const bool more = v + 1 <= v_hi;
      if (more) stage.issue(a, bt, g, tile(v + 1), pos);
      if (j0 + 16 * wave <= pos) {
        if (a.window_left < 0 && j0 + kTileKeys - 1 <= pos) attend_tile<D, DV, RB, 1, false>(w, sm[0], a, j0, wave);
        else attend_tile<D, DV, RB, 1, true>(w, sm[0], a, j0, wave);
      }
      __syncthreads();
      if (more) {
        stage.commit(sm[0]);
        __syncthreads();
      }
    }
  }
  constexpr int kRowF = DV + 4;
  float* lds = reinterpret_cast<float*>(&sm[0]);            // (the loop ended on a barrier: nobody reads the tiles any more)
  float lr[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float l = w.l[rb];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    lr[rb] = l;
  }
  // this wave's rows into LDS place `slot`, or (to == part) into the workspace
  auto put = [&](float* to, int rows_limit) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int r = 16 * rb + n;
      if (r >= rows_limit) continue;
      float* pr = to + r * kRowF;
      if (g4 == 0) pr[DV] = w.m[rb], pr[DV + 1] = lr[rb];
#pragma unroll
      for (int cb = 0; cb < DV / 16; ++cb) *reinterpret_cast<f32x4v*>(pr + 16 * cb + 4 * g4) = w.o[rb][cb];
    }
  };
  // another wave's rows from LDS merged into this wave's
  auto take = [&](const float* from) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const float* pr = from + (16 * rb + n) * kRowF;
      const float mp = pr[DV], lp = pr[DV + 1];
      const float m = fmaxf(w.m[rb], mp);
      const float f = w.m[rb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(w.m[rb] - m);      // (a wave that saw no key of the row)
      const float fp = mp == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mp - m);
#pragma unroll
      for (int cb = 0; cb < DV / 16; ++cb) w.o[rb][cb] = w.o[rb][cb] * f + *reinterpret_cast<const f32x4v*>(pr + 16 * cb + 4 * g4) * fp;
      lr[rb] = lr[rb] * f + lp * fp;
      w.m[rb] = m;
    }
  };
  if constexpr (kMerge) {
    static_assert(kDecodeWaves == 4, "the merge is a tree over four waves");
    if (wave >= 2) put(lds + (wave - 2) * 16 * RB * kRowF, 16 * RB);
    __syncthreads();
    if (wave < 2) take(lds + wave * 16 * RB * kRowF);
    __syncthreads();
    if (wave == 1) put(lds, 16 * RB);
    __syncthreads();
    if (wave == 0) {
      take(lds);
      put(part, HG);
    }
  } else {
    put(part, HG);
  }
}

// grid = (sequences, heads), 64 threads: merge the slices of a decode row, add the sink, normalise, store bf16.
__global__ __launch_bounds__(64) void sink_attention_decode_combine_kernel(hymeta_sink_attention_args a, int splits, ValueSlice vs) {
  // (splits: partials per (sequence, key/value head): one per slice, or one per wave of a slice)
  const int s = blockIdx.x;
  const int t = a.query_start_loc[s];
  if (a.query_start_loc[s + 1] - t != 1) return;
  const int group = a.num_heads / a.num_kv_heads, HG = vs.h_count ? vs.h_count : group;
  const int g = blockIdx.y / HG, r = blockIdx.y % HG, h = g * group + vs.h_first + r, DV = a.v_dim;
  const size_t stride = HG * partial_row_floats(DV);
  const float* base = static_cast<const float*>(a.workspace) + (static_cast<size_t>(s) * a.num_kv_heads + g) * splits * stride +
                      r * partial_row_floats(DV);
  // (the partials' maxima are in the base-2 domain, as the waves kept them)
  const float sink2 = a.sink_logits ? a.sink_logits[h] * 1.4426950408889634f : 0.f;
  float m = a.sink ? sink2 : -INFINITY;
  for (int sp = 0; sp < splits; ++sp) m = fmaxf(m, base[sp * stride + DV]);
  float l = a.sink ? __builtin_amdgcn_exp2f(sink2 - m) : 0.f;
  for (int sp = 0; sp < splits; ++sp) {
    const float ms = base[sp * stride + DV];
    if (ms != -INFINITY) l += base[sp * stride + DV + 1] * __builtin_amdgcn_exp2f(ms - m);
  }
  float inv = l > 0.f ? 1.f / l : 0.f;
  if (a.head_gate) inv *= sigmoid_exact(bf2f(static_cast<const uint16_t*>(a.head_gate)[static_cast<int64_t>(t) * a.head_gate_stride_t + h]));
  uint16_t* out = static_cast<uint16_t*>(a.out) + (static_cast<int64_t>(t) * a.num_heads + h) * vs.total + vs.first;
  for (int c = threadIdx.x; c < DV; c += 64) {
    float acc = 0.f;
    for (int sp = 0; sp < splits; ++sp) {
      const float ms = base[sp * stride + DV];
      if (ms != -INFINITY) acc += base[sp * stride + c] * __builtin_amdgcn_exp2f(ms - m);
    }
    out[c] = f2bf(acc * inv);
  }
}

// Head sizes the matrix-core kernels are built for.  A value inside its key: a latent of 64 or 128 followed by a rotated
// part of 32 or 64, or a latent of 256 / 384 / 512 followed by a rotated part of 64, which runs as 2 / 3 / 4 launches
// over value slices of 128 (each repeats the scores over the whole key: 1.5 to 2.1 times the matrix work of one pass
// with accumulators for all the value columns, which do not fit a wave's registers beside the query fragments).
inline bool mfma_shape(const hymeta_sink_attention_args& a) {
  bool dims = (a.head_dim == 64 || a.head_dim == 128) && (a.v_dim == 64 || a.v_dim == 128);
  if (a.kv_layout == HYMETA_KV_VALUE_IN_KEY)
    dims = ((a.v_dim == 64 || a.v_dim == 128) && (a.head_dim == a.v_dim + 32 || a.head_dim == a.v_dim + 64)) ||
           ((a.v_dim == 256 || a.v_dim == 384 || a.v_dim == 512) && a.head_dim == a.v_dim + 64);      // (in value slices of 128)
  // one key for all heads: the concatenated keys of 1 / 2 / 4 / 8 key/value heads of 64 or 128
  if (a.kv_layout == HYMETA_KV_SHARED_KEY)
    dims = (a.head_dim == 64 || a.head_dim == 128 || a.head_dim == 256 || a.head_dim == 512) && (a.v_dim == 64 || a.v_dim == 128);
  return a.act_dtype == HYMETA_BF16 && dims && a.q_stride_t % 8 == 0 &&
         (a.block_size & (a.block_size - 1)) == 0 &&
         (reinterpret_cast<uintptr_t>(a.q) | reinterpret_cast<uintptr_t>(a.kv_cache) | reinterpret_cast<uintptr_t>(a.out)) % 16 == 0;
}

inline int decode_splits(int num_seqs, int num_heads, int num_kv_heads, int max_seq_len) {
  const int tiles = (max_seq_len + kTileKeys - 1) / kTileKeys;
  // Workgroups aimed at: a workgroup's fixed cost (query fragments, first tile, the merge of its waves, its partial) grows
  // with the query heads it carries, so fewer, longer workgroups pay.  Measured at 64 sequences x 4096 keys: 28 heads on
  // one row of 192: 93 / 67 / 56 / 87 us at 1024 / 512 / 256 / 128; 16 heads on it: 53 / 40 / 45; 4 key/value heads with
  // 7 query heads each: 125 / 114 / 168.
  const int target = num_heads / num_kv_heads > 16 ? 256 : 512;
  int splits = (target + num_seqs * num_kv_heads - 1) / (num_seqs * num_kv_heads);
  splits = splits < 1 ? 1 : splits;
  return splits > tiles ? (tiles < 1 ? 1 : tiles) : splits;
}

template <int D, int DV, int Layout = HYMETA_KV_KEY_THEN_VALUE>
int launch_mfma(const hymeta_sink_attention_args& a, hipStream_t st, ValueSlice vs = ValueSlice{0, DV, 0, 0}) {
  if (a.max_query_len > 1) {
    constexpr int kRB = PREFILL_RB;
    constexpr int kRows = PrefillShape<kRB, PrefillWaves<D>::value>::kRows;
    const dim3 grid((a.max_query_len + kRows - 1) / kRows, a.num_heads, a.num_seqs);
    hipLaunchKernelGGL((sink_attention_prefill_mfma_kernel<D, DV, kRB, Layout>), grid, dim3(64 * PrefillWaves<D>::value), 0, st, a, vs);
  }
  // sequences with a single row: every step but a pure prompt step has some; a prompt of one token is one too
  const int splits = decode_splits(a.num_seqs, a.num_heads, a.num_kv_heads, a.max_seq_len);
  const int tiles = (a.max_seq_len + kTileKeys - 1) / kTileKeys;
  const int tiles_per_split = (tiles + splits - 1) / splits;
  const dim3 grid = Layout == HYMETA_KV_SHARED_KEY ? dim3((splits * a.num_seqs + 7) / 8 * 8 * a.num_kv_heads) : dim3(splits, a.num_kv_heads, a.num_seqs);
  const int group = a.num_heads / a.num_kv_heads;
  for (int first = 0; first < group; first += kRowsPerWave) {
    vs.h_first = first;
    vs.h_count = group - first < kRowsPerWave ? group - first : kRowsPerWave;
    int parts;
    if (vs.h_count <= 16) {
      hipLaunchKernelGGL((sink_attention_decode_mfma_kernel<D, DV, 1, Layout>), grid, dim3(64 * kDecodeWaves), 0, st, a, splits, tiles_per_split, vs);
      parts = splits * (DecodeMerge<D, DV, 1>::value ? 1 : kDecodeWaves);
    } else {
      hipLaunchKernelGGL((sink_attention_decode_mfma_kernel<D, DV, 2, Layout>), grid, dim3(64 * kDecodeWaves), 0, st, a, splits, tiles_per_split, vs);
      parts = splits * (DecodeMerge<D, DV, 2>::value ? 1 : kDecodeWaves);
    }
    hipLaunchKernelGGL(sink_attention_decode_combine_kernel, dim3(a.num_seqs, a.num_kv_heads * vs.h_count), dim3(64), 0, st, a, parts, vs);
  }
  return launch_status();
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_qk_norm_cache(const hymeta_qk_norm_cache_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_qk_norm_cache_args& a = *args;
  if (a.num_tokens < 0 || a.num_heads <= 0 || a.num_kv_heads <= 0 || a.head_dim <= 0 || a.v_dim <= 0 || a.block_size <= 0 ||
      a.num_blocks < 0)
    return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.qkv || (a.slot_mapping && !a.kv_cache)) return HYMETA_ERR_INVALID_ARG;
  if (a.qkv_stride_t < static_cast<int64_t>(a.num_heads + a.num_kv_heads) * a.head_dim + static_cast<int64_t>(a.num_kv_heads) * a.v_dim)
    return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(qk_norm_cache_kernel<ActBf16>, dim3(a.num_tokens), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(qk_norm_cache_kernel<ActF32>, dim3(a.num_tokens), dim3(256), 0, st, a);
  return launch_status();
}

extern "C" size_t hymeta_sink_attention_workspace_bytes(int32_t num_seqs, int32_t num_heads, int32_t num_kv_heads, int32_t v_dim,
                                                        int32_t max_seq_len) {
  if (num_seqs <= 0 || num_heads <= 0 || num_kv_heads <= 0 || v_dim <= 0) return 0;
  const int splits = decode_splits(num_seqs, num_heads, num_kv_heads, max_seq_len < 1 ? 1 : max_seq_len);
  return static_cast<size_t>(num_seqs) * splits * kDecodeWaves * num_heads * partial_row_floats(v_dim) * sizeof(float);
}

extern "C" int hymeta_sink_attention(const hymeta_sink_attention_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_sink_attention_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.num_heads <= 0 || a.num_kv_heads <= 0 || a.head_dim <= 0 || a.v_dim <= 0 ||
      a.block_size <= 0 || a.num_blocks < 0)
    return HYMETA_ERR_INVALID_ARG;
  if (a.num_heads % a.num_kv_heads != 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.head_dim > kMaxHeadDim || a.v_dim > 64 * kMaxVChunks) return HYMETA_ERR_UNSUPPORTED;
  if (a.bias_mode != HYMETA_BIAS_NONE && a.bias_mode != HYMETA_BIAS_LOG_DISTANCE) return HYMETA_ERR_UNSUPPORTED;
  if (a.kv_layout != HYMETA_KV_KEY_THEN_VALUE && a.kv_layout != HYMETA_KV_VALUE_IN_KEY && a.kv_layout != HYMETA_KV_SHARED_KEY) return HYMETA_ERR_UNSUPPORTED;
  if (a.window_left >= 0 && a.keep_first < 0) return HYMETA_ERR_INVALID_ARG;
  if (a.kv_layout == HYMETA_KV_VALUE_IN_KEY && a.v_dim > a.head_dim) return HYMETA_ERR_INVALID_ARG;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.q || !a.kv_cache || !a.out || !a.block_tables || !a.query_start_loc || !a.seq_lens) return HYMETA_ERR_INVALID_ARG;
  if (a.bias_mode != HYMETA_BIAS_NONE && (!a.bias_a || !a.bias_b)) return HYMETA_ERR_INVALID_ARG;
  if (a.softcap < 0.f || (a.head_gate && a.head_gate_stride_t < a.num_heads)) return HYMETA_ERR_INVALID_ARG;
  if (a.num_heads > 65535) return HYMETA_ERR_UNSUPPORTED;
  hipStream_t st = begin_launches(stream);
  if (mfma_shape(a) && a.max_query_len >= 1 && a.max_seq_len >= 1) {
    const size_t need = hymeta_sink_attention_workspace_bytes(a.num_seqs, a.num_heads, a.num_kv_heads, a.v_dim, a.max_seq_len);
    if (!a.workspace || a.workspace_bytes < need) return HYMETA_ERR_WORKSPACE;
    if (a.num_seqs > 65535 || a.num_heads > 65535) return HYMETA_ERR_UNSUPPORTED;
    if (a.kv_layout == HYMETA_KV_VALUE_IN_KEY) {
      if (a.v_dim == 64) return a.head_dim == 96 ? launch_mfma<96, 64, HYMETA_KV_VALUE_IN_KEY>(a, st) : launch_mfma<128, 64, HYMETA_KV_VALUE_IN_KEY>(a, st);
      if (a.v_dim == 128) return a.head_dim == 160 ? launch_mfma<160, 128, HYMETA_KV_VALUE_IN_KEY>(a, st) : launch_mfma<192, 128, HYMETA_KV_VALUE_IN_KEY>(a, st);
      hymeta_sink_attention_args b = a;
      b.v_dim = 128;
      for (int first = 0; first < a.v_dim; first += 128) {
        const ValueSlice vs{first, a.v_dim, 0, 0};
        const int rc = a.v_dim == 256 ? launch_mfma<320, 128, HYMETA_KV_VALUE_IN_KEY>(b, st, vs) : a.v_dim == 384 ? launch_mfma<448, 128, HYMETA_KV_VALUE_IN_KEY>(b, st, vs)
                                                                                                 : launch_mfma<576, 128, HYMETA_KV_VALUE_IN_KEY>(b, st, vs);
        if (rc != HYMETA_OK) return rc;
      }
      return HYMETA_OK;
    }
    if (a.kv_layout == HYMETA_KV_SHARED_KEY) {
      constexpr int kShared = HYMETA_KV_SHARED_KEY;
      if (a.v_dim == 64)
        return a.head_dim == 64 ? launch_mfma<64, 64, kShared>(a, st) : a.head_dim == 128 ? launch_mfma<128, 64, kShared>(a, st)
             : a.head_dim == 256 ? launch_mfma<256, 64, kShared>(a, st) : launch_mfma<512, 64, kShared>(a, st);
      return a.head_dim == 64 ? launch_mfma<64, 128, kShared>(a, st) : a.head_dim == 128 ? launch_mfma<128, 128, kShared>(a, st)
           : a.head_dim == 256 ? launch_mfma<256, 128, kShared>(a, st) : launch_mfma<512, 128, kShared>(a, st);
    }
    if (a.head_dim == 64 && a.v_dim == 64) return launch_mfma<64, 64>(a, st);
    if (a.head_dim == 64 && a.v_dim == 128) return launch_mfma<64, 128>(a, st);
    if (a.head_dim == 128 && a.v_dim == 64) return launch_mfma<128, 64>(a, st);
    return launch_mfma<128, 128>(a, st);
  }
  const dim3 grid(a.num_tokens, a.num_heads);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(sink_attention_rows_kernel<ActBf16>, grid, dim3(64), 0, st, a);
  else hipLaunchKernelGGL(sink_attention_rows_kernel<ActF32>, grid, dim3(64), 0, st, a);
  return launch_status();
}
