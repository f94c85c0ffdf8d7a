// Glue of parallel-layer designs (one norm, mixer and feed-forward side by side on an fp32 stream): the sum of a
// layer's outputs onto the stream with the next layer's scalar-weight RMS norm; the rotate-half rotation of a fused
// projection's queries and keys with the paged key / value write; and the short causal convolution (bias, silu) of a
// state-space layer with its step sizes.  act_dtype in and out, fp32 inside.
#include "act_types.h"

namespace hymeta {

namespace {

// ------------------------------------------------------------------------------------------------ stream add + norm
constexpr int kAddVecs = 4;                  // rows up to 256 * 4 * kAddVecs columns stay in registers between the sum and the norm

// Vec: a thread takes runs of four consecutive columns (one load per term and run) and keeps them for the norm; otherwise
// column by column, the stream read again for the norm.
template <typename A, bool Vec>
__global__ __launch_bounds__(256) void stream_add_norm_kernel(hymeta_stream_add_norm_args a) {
  typedef typename A::elem elem;
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  float* x = a.x + t * a.x_stride_t;
  float scale[HYMETA_STREAM_MAX_TERMS];
  const elem* y[HYMETA_STREAM_MAX_TERMS];
#pragma unroll
  for (int i = 0; i < HYMETA_STREAM_MAX_TERMS; ++i) {
    const bool on = i < a.num_terms;
    scale[i] = on ? a.coef[i] * (a.row_scale[i] ? a.row_scale[i][t] : 1.f) : 0.f;
    y[i] = on ? static_cast<const elem*>(a.y[i]) + t * a.y_stride_t[i] : nullptr;
  }
  elem* h = a.h_out ? static_cast<elem*>(a.h_out) + t * a.width : nullptr;
  float ss = 0.f;
  if (Vec) {
    float v[kAddVecs][4];
#pragma unroll
    for (int u = 0; u < kAddVecs; ++u) {
      const int c = 4 * (threadIdx.x + 256 * u);
      if (c >= a.width) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[u][e] = 0.f;
        continue;
      }
      const f32x4 xv = *reinterpret_cast<const f32x4*>(x + c);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[u][e] = xv[e];
#pragma unroll
      for (int i = 0; i < HYMETA_STREAM_MAX_TERMS; ++i) {
        if (i < a.num_terms) {
          float yv[4];
          A::ld4(y[i] + c, yv);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[u][e] = fmaf(scale[i], yv[e], v[u][e]);
        }
      }
      if (a.num_terms > 0) *reinterpret_cast<f32x4*>(x + c) = f32x4{v[u][0], v[u][1], v[u][2], v[u][3]};
#pragma unroll
      for (int e = 0; e < 4; ++e) ss = fmaf(v[u][e], v[u][e], ss);
    }
    if (h == nullptr) return;
    ss = block_sum<4>(ss, red);
    const float inv = a.norm_scale / sqrtf(ss / static_cast<float>(a.width) + a.eps);
#pragma unroll
    for (int u = 0; u < kAddVecs; ++u) {
      const int c = 4 * (threadIdx.x + 256 * u);
      if (c >= a.width) continue;
      float o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = v[u][e] * inv * (a.norm_weight ? a.norm_weight[c + e] : 1.f);
      A::st4(h + c, o);
    }
    return;
  }
  for (int c = threadIdx.x; c < a.width; c += 256) {
    float v = x[c];
#pragma unroll
    for (int i = 0; i < HYMETA_STREAM_MAX_TERMS; ++i)
      if (i < a.num_terms) v = fmaf(scale[i], A::ld(y[i] + c), v);
    if (a.num_terms > 0) x[c] = v;
    ss = fmaf(v, v, ss);
  }
  if (h == nullptr) return;
  ss = block_sum<4>(ss, red);
  const float inv = a.norm_scale / sqrtf(ss / static_cast<float>(a.width) + a.eps);
  for (int c = threadIdx.x; c < a.width; c += 256) A::st(h + c, x[c] * inv * (a.norm_weight ? a.norm_weight[c] : 1.f));
}

// ------------------------------------------------------------------------------------------------ rotate half + cache
constexpr int kMaxRotPairs = 512;

// grid = tokens, 256 threads.  Work items of a token: a (head, pair) of the rotated dimensions of a query or key head, a
// passing dimension of a key head (scaled, stored), or a value element (stored).  A pair is read and written by one thread.
template <typename A>
__global__ __launch_bounds__(256) void rotary_cache_kernel(hymeta_rotary_cache_args a) {
  typedef typename A::elem elem;
  __shared__ float s_cos[kMaxRotPairs], s_sin[kMaxRotPairs];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int H = a.num_heads, G = a.num_kv_heads, D = a.head_dim, Dv = a.v_dim, half = a.rot_dims / 2;
  int pos;
  if (a.positions) {
    pos = static_cast<int>(a.positions[t]);
  } else {
    const int s = seq_of_row(a.query_start_loc, a.num_seqs, t);
    pos = max(a.seq_lens[s] - (a.query_start_loc[s + 1] - t), 0);
  }
  // angles in double precision, brought into [-pi, pi]; the functions are the fp32 ones on the remainder
  for (int i = tid; i < half; i += 256) {
    constexpr double kTwoPi = 6.283185307179586476925286766559, kInvTwoPi = 0.15915494309189533576888376337251;
    const double ang = static_cast<double>(pos) * a.rot_freqs[i];
    const float r = static_cast<float>(fma(-kTwoPi, rint(ang * kInvTwoPi), ang));
    s_cos[i] = cosf(r);
    s_sin[i] = sinf(r);
  }
  __syncthreads();
  elem* row = static_cast<elem*>(a.qkv) + static_cast<int64_t>(t) * a.qkv_stride_t;
  const int64_t slot = a.slot_mapping ? a.slot_mapping[t] : -1;
  const bool store = a.kv_cache != nullptr && slot >= 0 && slot < a.num_blocks * a.block_size;
  elem* cache = store ? static_cast<elem*>(a.kv_cache) + slot * G * static_cast<int64_t>(D + Dv) : nullptr;
  const float ks = a.k_scale != 0.f ? a.k_scale : 1.f;
  // per head: `half` pairs, then the D - 2 half passing dimensions
  const int per_head = D - half;
  for (int w = tid; w < (H + G) * per_head; w += 256) {
    const int head = w / per_head, i = w % per_head;
    const bool is_q = head < H;
    elem* src = row + static_cast<int64_t>(head) * D;
    elem* dst = is_q ? nullptr : (cache ? cache + static_cast<int64_t>(head - H) * (D + Dv) : nullptr);
    const float mul = is_q ? 1.f : ks;
    if (i < half) {
      const float u = A::ld(src + i), v = A::ld(src + i + half), c = s_cos[i], sn = s_sin[i];
      const float ru = (u * c - v * sn) * mul, rv = (v * c + u * sn) * mul;
      A::st(src + i, ru);
      A::st(src + i + half, rv);
      if (dst) {
        A::st(dst + i, ru);
        A::st(dst + i + half, rv);
      }
    } else {
      const int d = half + i;               // dimensions 2 half .. D - 1
      if (is_q) continue;
      const float v = A::ld(src + d) * mul;
      if (mul != 1.f) A::st(src + d, v);
      if (dst) A::st(dst + d, v);
    }
  }
  if (cache) {
    const elem* vsrc = row + static_cast<int64_t>(H + G) * D;
    for (int w = tid; w < G * Dv; w += 256) {
      const int g = w / Dv, d = w % Dv;
      cache[static_cast<int64_t>(g) * (D + Dv) + D + d] = vsrc[w];
    }
  }
}

// ------------------------------------------------------------------------------------------------ causal convolution
__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

// grid = (tokens, channel runs of 256): a thread computes one channel of one row from the row and its taps - 1
// predecessors (rows of the step, or the sequence's state).  The first run's workgroup also computes the row's step sizes.
// SingleRows: every sequence brings one row (row t is sequence t's), and the thread that read its channel of the state
// also moves it on by the row -- a decode step's convolution in one launch.
template <typename A, bool SingleRows>
__global__ __launch_bounds__(256) void causal_conv_kernel(hymeta_causal_conv_args a) {
  typedef typename A::elem elem;
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  const int s = SingleRows ? t : seq_of_row(a.query_start_loc, a.num_seqs, t);
  const int r0 = a.query_start_loc[s], i = t - r0, hist = a.taps - 1;
  if (blockIdx.y == 0 && a.dt_in != nullptr && threadIdx.x < a.dt_heads) {
    const int h = threadIdx.x;
    for (int hh = h; hh < a.dt_heads; hh += 256) {
      const float raw = A::ld(static_cast<const elem*>(a.dt_in) + static_cast<int64_t>(t) * a.dt_stride_t + hh);
      const float dt = softplus_f(raw + a.dt_bias[hh]);
      a.dt_out[static_cast<int64_t>(t) * a.dt_heads + hh] = dt;
      a.log2_decay_out[static_cast<int64_t>(t) * a.dt_heads + hh] = -expf(a.a_log[hh]) * dt * 1.4426950408889634f;
    }
  }
  if (c >= a.channels) return;
  const int slot = a.slot_idx ? a.slot_idx[s] : -1;
  elem* own = (a.conv_state && slot >= 0) ? static_cast<elem*>(a.conv_state) + static_cast<int64_t>(slot) * hist * a.channels : nullptr;
  const elem* state = a.context_lens[s] > 0 ? own : nullptr;
  const elem* x = static_cast<const elem*>(a.x);
  float acc = a.bias ? a.bias[c] : 0.f;
  elem taps_in[HYMETA_CONV_MAX_TAPS];                 // the inputs as stored (what the state keeps)
  for (int j = 0; j < a.taps; ++j) {
    const int back = hist - j;                    // rows before t
    elem raw = static_cast<elem>(0);
    if (back <= i) raw = x[static_cast<int64_t>(t - back) * a.x_stride_t + c];
    else if (state) raw = state[static_cast<int64_t>(hist - (back - i)) * a.channels + c];       // state row hist - 1 is the newest
    taps_in[j] = raw;
    acc = fmaf(a.weight[static_cast<int64_t>(c) * a.taps + j], A::ld(&raw), acc);
  }
  A::st(static_cast<elem*>(a.out) + static_cast<int64_t>(t) * a.channels + c, acc * sigmoid_exact(acc));
  if (SingleRows && own != nullptr)
    for (int j = 0; j < hist; ++j) own[static_cast<int64_t>(j) * a.channels + c] = taps_in[j + 1];
}

// Many rows, channels in whole fours: a thread takes four consecutive channels through a strip of kConvRows rows, the
// weights and the last taps - 1 inputs in registers (an input row is read once per strip instead of once per tap); a strip
// may run over the end of a sequence into the next one, whose history it then fetches anew.
constexpr int kConvRows = 8;

template <typename A>
__global__ __launch_bounds__(256) void causal_conv_strip_kernel(hymeta_causal_conv_args a) {
  typedef typename A::elem elem;
  constexpr int MH = HYMETA_CONV_MAX_TAPS - 1;
  const int t0 = blockIdx.x * kConvRows, t1 = min(t0 + kConvRows, a.num_tokens);
  const int c = 4 * (blockIdx.y * 256 + threadIdx.x), hist = a.taps - 1;
  if (blockIdx.y == 0 && a.dt_in != nullptr) {
    for (int idx = threadIdx.x; idx < (t1 - t0) * a.dt_heads; idx += 256) {
      const int64_t t = t0 + idx / a.dt_heads;
      const int hh = idx % a.dt_heads;
      const float dt = softplus_f(A::ld(static_cast<const elem*>(a.dt_in) + t * a.dt_stride_t + hh) + a.dt_bias[hh]);
      a.dt_out[t * a.dt_heads + hh] = dt;
      a.log2_decay_out[t * a.dt_heads + hh] = -expf(a.a_log[hh]) * dt * 1.4426950408889634f;
    }
  }
  if (c >= a.channels) return;
  float w[HYMETA_CONV_MAX_TAPS][4], bias[4], past[MH][4];
#pragma unroll
  for (int j = 0; j < HYMETA_CONV_MAX_TAPS; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) w[j][e] = j < a.taps ? a.weight[static_cast<int64_t>(c + e) * a.taps + j] : 0.f;
#pragma unroll
  for (int e = 0; e < 4; ++e) bias[e] = a.bias ? a.bias[c + e] : 0.f;
  const elem* x = static_cast<const elem*>(a.x);
  int s = seq_of_row(a.query_start_loc, a.num_seqs, t0);
  int r0 = a.query_start_loc[s], r1 = a.query_start_loc[s + 1];
  // past[j]: the input hist - j rows before row t (the oldest first), from the step's rows, the sequence's state, or zeros
  auto fetch_past = [&](int t) {
    const int i = t - r0;
    const int slot = a.slot_idx ? a.slot_idx[s] : -1;
    const elem* state = (a.conv_state && slot >= 0 && a.context_lens[s] > 0)
                            ? static_cast<const elem*>(a.conv_state) + static_cast<int64_t>(slot) * hist * a.channels : nullptr;
#pragma unroll
    for (int j = 0; j < MH; ++j) {
#pragma unroll
      for (int e = 0; e < 4; ++e) past[j][e] = 0.f;
      if (j >= hist) continue;
      const int back = hist - j;
      if (back <= i) A::ld4(x + static_cast<int64_t>(t - back) * a.x_stride_t + c, past[j]);
      else if (state) A::ld4(state + static_cast<int64_t>(hist - (back - i)) * a.channels + c, past[j]);
    }
  };
  fetch_past(t0);
  for (int t = t0; t < t1; ++t) {
    if (t >= r1) {
      while (t >= r1) r1 = a.query_start_loc[++s + 1];
      r0 = a.query_start_loc[s];
      fetch_past(t);
    }
    float cur[4], acc[4];
    A::ld4(x + static_cast<int64_t>(t) * a.x_stride_t + c, cur);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = bias[e];
#pragma unroll
    for (int j = 0; j < MH; ++j)
      if (j < hist) {
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = fmaf(w[j][e], past[j][e], acc[e]);
      }
#pragma unroll
    for (int j = 0; j < HYMETA_CONV_MAX_TAPS; ++j)
      if (j == hist) {
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = fmaf(w[j][e], cur[e], acc[e]);
      }
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = acc[e] * sigmoid_exact(acc[e]);
    A::st4(static_cast<elem*>(a.out) + static_cast<int64_t>(t) * a.channels + c, acc);
    // the window moves on by a row (in ascending j: past[j + 1] is still the old one)
#pragma unroll
    for (int j = 0; j < MH; ++j) {
      constexpr int kLast = MH - 1;
      const int nxt = j < kLast ? j + 1 : kLast;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (j + 1 < hist) past[j][e] = past[nxt][e];
        else if (j + 1 == hist) past[j][e] = cur[e];
      }
    }
  }
}

// grid = (sequences, channel runs of 256): the state becomes the last taps - 1 input rows (older rows of the old state move
// up where the step brought fewer rows).  A thread reads all of its channel's old rows before it writes.
template <typename A>
__global__ __launch_bounds__(256) void causal_conv_state_kernel(hymeta_causal_conv_args a) {
  typedef typename A::elem elem;
  const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= a.channels) return;
  const int slot = a.slot_idx[s];
  if (slot < 0) return;
  const int r0 = a.query_start_loc[s], q = a.query_start_loc[s + 1] - r0, hist = a.taps - 1;
  if (q <= 0) return;
  elem* state = static_cast<elem*>(a.conv_state) + static_cast<int64_t>(slot) * hist * a.channels;
  const bool carried = a.context_lens[s] > 0;
  const elem* x = static_cast<const elem*>(a.x);
  elem keep[HYMETA_CONV_MAX_TAPS];
  for (int j = 0; j < hist; ++j) {
    // new state row j is the input hist - 1 - j rows before the step's last row
    const int back = hist - 1 - j;
    if (back < q) keep[j] = x[static_cast<int64_t>(r0 + q - 1 - back) * a.x_stride_t + c];
    else {
      const int old = j + q;                      // (back - q) rows before the old state's newest: row hist - 1 - (back - q)
      keep[j] = carried ? state[static_cast<int64_t>(old) * a.channels + c] : static_cast<elem>(0);
    }
  }
  for (int j = 0; j < hist; ++j) state[static_cast<int64_t>(j) * a.channels + c] = keep[j];
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_stream_add_norm(const hymeta_stream_add_norm_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_stream_add_norm_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0 || a.num_terms < 0 || a.num_terms > HYMETA_STREAM_MAX_TERMS) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.x || a.x_stride_t < a.width || (a.num_terms == 0 && !a.h_out)) return HYMETA_ERR_INVALID_ARG;
  for (int i = 0; i < a.num_terms; ++i)
    if (!a.y[i] || a.y_stride_t[i] < a.width) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  // runs of four: every pointer and stride in whole fours of its type, the row inside the registers
  const int eb = a.act_dtype == HYMETA_BF16 ? 2 : 4;
  bool cached = a.width % 4 == 0 && a.width <= 256 * 4 * kAddVecs && reinterpret_cast<uintptr_t>(a.x) % 16 == 0 && a.x_stride_t % 4 == 0 &&
                (!a.h_out || reinterpret_cast<uintptr_t>(a.h_out) % (4 * eb) == 0);
  for (int i = 0; i < a.num_terms; ++i) cached = cached && reinterpret_cast<uintptr_t>(a.y[i]) % (4 * eb) == 0 && a.y_stride_t[i] % 4 == 0;
  if (a.act_dtype == HYMETA_BF16) {
    if (cached) hipLaunchKernelGGL((stream_add_norm_kernel<ActBf16, true>), dim3(a.num_tokens), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((stream_add_norm_kernel<ActBf16, false>), dim3(a.num_tokens), dim3(256), 0, st, a);
  } else {
    if (cached) hipLaunchKernelGGL((stream_add_norm_kernel<ActF32, true>), dim3(a.num_tokens), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((stream_add_norm_kernel<ActF32, false>), dim3(a.num_tokens), dim3(256), 0, st, a);
  }
  return launch_status();
}

extern "C" int hymeta_rotary_cache(const hymeta_rotary_cache_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_rotary_cache_args& a = *args;
  if (a.num_tokens < 0 || a.num_heads <= 0 || a.num_kv_heads <= 0 || a.head_dim <= 0 || a.v_dim < 0 || a.num_blocks < 0) return HYMETA_ERR_INVALID_ARG;
  if (a.rot_dims < 0 || a.rot_dims % 2 != 0 || a.rot_dims > a.head_dim) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.rot_dims / 2 > kMaxRotPairs) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.qkv || (a.rot_dims > 0 && !a.rot_freqs)) return HYMETA_ERR_INVALID_ARG;
  if (a.rot_dims > 0 && !a.positions && (!a.query_start_loc || !a.seq_lens || a.num_seqs <= 0)) return HYMETA_ERR_INVALID_ARG;
  if (a.kv_cache && (!a.slot_mapping || a.block_size <= 0)) return HYMETA_ERR_INVALID_ARG;
  if (a.qkv_stride_t < static_cast<int64_t>(a.num_heads + a.num_kv_heads) * a.head_dim + (a.kv_cache ? static_cast<int64_t>(a.num_kv_heads) * a.v_dim : 0))
    return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(rotary_cache_kernel<ActBf16>, dim3(a.num_tokens), dim3(256), 0, st, a);
  else hipLaunchKernelGGL(rotary_cache_kernel<ActF32>, dim3(a.num_tokens), dim3(256), 0, st, a);
  return launch_status();
}

extern "C" int hymeta_causal_conv(const hymeta_causal_conv_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_causal_conv_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.channels <= 0 || a.dt_heads < 0) return HYMETA_ERR_INVALID_ARG;
  if (a.taps < 1 || a.taps > HYMETA_CONV_MAX_TAPS) return HYMETA_ERR_UNSUPPORTED;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.x || !a.weight || !a.out || !a.query_start_loc || !a.context_lens || a.x_stride_t < a.channels) return HYMETA_ERR_INVALID_ARG;
  if (a.conv_state && !a.slot_idx) return HYMETA_ERR_INVALID_ARG;
  if (a.dt_in && (!a.dt_bias || !a.a_log || !a.dt_out || !a.log2_decay_out || a.dt_stride_t < a.dt_heads)) return HYMETA_ERR_INVALID_ARG;
  const int runs = (a.channels + 255) / 256;
  if (runs > 65535 || a.num_seqs > 65535) return HYMETA_ERR_UNSUPPORTED;
  hipStream_t st = begin_launches(stream);
  const bool bf = a.act_dtype == HYMETA_BF16;
  const int eb = bf ? 2 : 4;
  const bool fours = a.channels % 4 == 0 && a.x_stride_t % 4 == 0 && reinterpret_cast<uintptr_t>(a.x) % (4 * eb) == 0 &&
                     reinterpret_cast<uintptr_t>(a.out) % (4 * eb) == 0 && (!a.conv_state || reinterpret_cast<uintptr_t>(a.conv_state) % (4 * eb) == 0);
  if (a.num_tokens == a.num_seqs && a.single_rows) {
    if (bf) hipLaunchKernelGGL((causal_conv_kernel<ActBf16, true>), dim3(a.num_tokens, runs), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((causal_conv_kernel<ActF32, true>), dim3(a.num_tokens, runs), dim3(256), 0, st, a);
    return launch_status();
  }
  // strips pay once there are rows enough to fill the chip with a quarter of the threads
  if (fours && a.num_tokens >= 32 * kConvRows) {
    const dim3 grid((a.num_tokens + kConvRows - 1) / kConvRows, (a.channels / 4 + 255) / 256);
    if (bf) hipLaunchKernelGGL(causal_conv_strip_kernel<ActBf16>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(causal_conv_strip_kernel<ActF32>, grid, dim3(256), 0, st, a);
  } else {
    if (bf) hipLaunchKernelGGL((causal_conv_kernel<ActBf16, false>), dim3(a.num_tokens, runs), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((causal_conv_kernel<ActF32, false>), dim3(a.num_tokens, runs), dim3(256), 0, st, a);
  }
  if (a.conv_state && a.taps > 1) {
    if (bf) hipLaunchKernelGGL(causal_conv_state_kernel<ActBf16>, dim3(a.num_seqs, runs), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(causal_conv_state_kernel<ActF32>, dim3(a.num_seqs, runs), dim3(256), 0, st, a);
  }
  return launch_status();
}
