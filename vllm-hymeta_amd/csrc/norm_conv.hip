// fp32 residual stream: embedding rows, RMS norm (+ short causal convolution over time with a carried
// state) on the way into a sublayer, output norm + scaled residual add on the way out.
//
// The norm statistics and the convolution are fp32; the normed row is rounded to the activation type
// before the convolution reads it (it is what a norm kernel on its own would have stored, and what the
// carried state holds), so a row's value does not depend on whether its predecessors came from this
// step or from the state.
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kNormThreads = 256;
constexpr int kNormWaves = kNormThreads / 64;
constexpr int kMaxPerThread = 32;          // width <= 256 * 32 channels

template <typename A>
__global__ __launch_bounds__(kNormThreads) void embed_rows_kernel(hymeta_embed_rows_args a) {
  const int t = blockIdx.x;
  int64_t tok = a.token_ids[t];
  if (tok < 0 || tok >= a.vocab) tok = 0;          // ids are validated on the host; never read out of the table
  const typename A::elem* row = static_cast<const typename A::elem*>(a.table) + tok * a.width;
  float* out = a.out + static_cast<int64_t>(t) * a.width;
  const float scale = a.scale != 0.f ? a.scale : 1.f;
  for (int c = threadIdx.x; c < a.width; c += kNormThreads) out[c] = A::ld(row + c) * scale + (a.add ? a.add[c] : 0.f);
}

__device__ __forceinline__ int seq_of_row_fast(const hymeta_norm_conv_args& a, int t);

constexpr int kMaxRows = 2 * (HYMETA_CONV_MAX_TAPS - 1);
constexpr int kRowUnroll = 16;               // channels per thread whose loads are issued together (width <= 4096)      // rows whose statistic one workgroup may need

// One workgroup per token row.  Rows 1 .. taps - 2 of a portion are computed by the workgroup of its row 0, which is
// also the only one that touches the sequence's convolution state: it reads the old rows for the portion's first
// outputs and then writes the new ones.  A thread owns its channels in all of this, so no other thread waits for its
// reads or sees its writes.  The sums of squares of all the rows a workgroup needs (its own and its predecessors',
// for the first workgroup also the rows that become the new state) are reduced together, one barrier pair.
template <typename A>
__device__ __forceinline__ void norm_conv_row(const hymeta_norm_conv_args& a, int t, float (*red)[kMaxRows]) {
  typedef typename A::elem elem;
  const int taps = a.conv_weight ? a.taps : 1;
  const int hist = taps - 1;
  int s = 0, i = 0, q = 1, ctx = 0, slot = -1;
  int64_t row0 = t;
  if (hist > 0) {
    // a step of single rows (decode) has sequence t at row t: two independent loads instead of a search
    s = seq_of_row_fast(a, t);
    row0 = a.query_start_loc[s];
    i = t - static_cast<int>(row0);
    q = a.query_start_loc[s + 1] - static_cast<int>(row0);
    ctx = a.context_lens[s];
    slot = a.slot_idx ? a.slot_idx[s] : -1;
    if (i > 0 && i < hist) return;                     // computed by the portion's first workgroup
  }
  elem* state = (hist > 0 && a.conv_state && slot >= 0)
                    ? static_cast<elem*>(a.conv_state) + static_cast<int64_t>(slot) * hist * a.width : nullptr;
  const bool carried = state != nullptr && ctx > 0;
  const bool first = hist > 0 && i == 0;
  const int todo = first ? min(hist, q) : 1;

  // portion rows whose statistic is needed: [lo1, lo1 + n1) for the outputs, [lo2, lo2 + n2) more for the new state
  const int lo1 = first ? 0 : i - hist, n1 = first ? todo : taps;
  const int lo2 = max(todo, q - hist), n2 = (first && state != nullptr) ? max(0, q - lo2) : 0;
  float ss[kMaxRows];
#pragma unroll
  for (int r = 0; r < kMaxRows; ++r) ss[r] = 0.f;
  // (the first 16 channels of a thread with every load in flight at once; wider rows go on in a plain loop)
  auto stats_at = [&](int c) {
#pragma unroll
    for (int r = 0; r < kMaxRows; ++r) {
      if (r < n1 + n2) {
        const int k = r < n1 ? lo1 + r : lo2 + (r - n1);
        const float v = a.x[(row0 + k) * a.x_stride_t + c];
        ss[r] = fmaf(v, v, ss[r]);
      }
    }
  };
#pragma unroll
  for (int u = 0; u < kRowUnroll; ++u) {
    const int c = threadIdx.x + u * kNormThreads;
    if (c < a.width) stats_at(c);
  }
  for (int c = threadIdx.x + kRowUnroll * kNormThreads; c < a.width; c += kNormThreads) stats_at(c);
#pragma unroll
  for (int r = 0; r < kMaxRows; ++r)
    if (r < n1 + n2) {
      const float v = wave_sum(ss[r]);
      if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6][r] = v;
    }
  __syncthreads();
  float inv[kMaxRows];
#pragma unroll
  for (int r = 0; r < kMaxRows; ++r) {
    inv[r] = 0.f;
    if (r < n1 + n2) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < kNormWaves; ++w) v += red[w][r];
      inv[r] = 1.f / sqrtf(v / static_cast<float>(a.width) + a.eps);
    }
  }
  // the statistic of portion row k (k in one of the two ranges)
  auto inv_of = [&](int k) -> float {
    const int r = (k >= lo1 && k < lo1 + n1) ? k - lo1 : n1 + (k - lo2);
    float v = 0.f;
#pragma unroll
    for (int u = 0; u < kMaxRows; ++u) v = (u == r) ? inv[u] : v;
    return v;
  };

  auto emit_at = [&](int c) {
    const float w = a.weight_offset + a.weight[c];
    const float* cw = a.conv_weight ? a.conv_weight + static_cast<int64_t>(c) * taps : nullptr;
    // the normed value of portion row k of this channel (k < 0: from the carried state, or zero)
    auto normed = [&](int k) -> float {
      if (k >= 0) return A::round(a.x[(row0 + k) * a.x_stride_t + c] * inv_of(k) * w);
      return carried ? A::ld(state + static_cast<int64_t>(hist + k) * a.width + c) : 0.f;
    };
    for (int ii = i; ii < i + todo; ++ii) {
      const float n = normed(ii);
      float acc = n;
      if (cw != nullptr) {
        acc = fmaf(cw[hist], n, acc);
        for (int j = 0; j < hist; ++j) acc = fmaf(cw[j], normed(ii - hist + j), acc);
      }
      A::st(static_cast<elem*>(a.out) + (row0 + ii) * static_cast<int64_t>(a.width) + c, acc);
    }
    if (first && state != nullptr) {
      // new state row r = the normed row at portion index q - hist + r; indices before the portion come from the old
      // state (row q + r, which lies after the row being written: ascending r never reads a row already replaced)
      for (int r = 0; r < hist; ++r) A::st(state + static_cast<int64_t>(r) * a.width + c, normed(q - hist + r));
    }
  };
#pragma unroll
  for (int u = 0; u < kRowUnroll; ++u) {
    const int c = threadIdx.x + u * kNormThreads;
    if (c < a.width) emit_at(c);
  }
  for (int c = threadIdx.x + kRowUnroll * kNormThreads; c < a.width; c += kNormThreads) emit_at(c);
}

// Sequence of row t, with the shortcut for steps of single rows (sequence t at row t).
__device__ __forceinline__ int seq_of_row_fast(const hymeta_norm_conv_args& a, int t) {
  if (t < a.num_seqs && a.query_start_loc[t] == t && a.query_start_loc[t + 1] == t + 1) return t;
  return seq_of_row(a.query_start_loc, a.num_seqs, t);
}

constexpr int kStripHist = 3;                  // the strip form covers taps <= 4 ...
constexpr int kStripPerThread = 16;            // ... and width <= 256 * 16

// A workgroup per strip of R consecutive rows.  Where the strip lies inside one portion, past the rows that read the
// carried state, its R + taps - 1 input rows are read once into registers, their statistics reduced together, and every
// output row takes its predecessors from the registers; other strips (a portion's first rows, strips over a boundary
// between sequences) go row by row through norm_conv_row.
template <typename A, int R>
__global__ __launch_bounds__(kNormThreads) void norm_conv_kernel(hymeta_norm_conv_args a) {
  typedef typename A::elem elem;
  __shared__ float red[kNormWaves][kMaxRows];
  const int t0 = blockIdx.x * R;
  const int rows = min(R, a.num_tokens - t0);
  const int taps = a.conv_weight ? a.taps : 1;
  const int hist = taps - 1;
  bool strip = false;
  if (R > 1 && hist > 0 && hist <= kStripHist && rows == R && a.width <= kNormThreads * kStripPerThread) {
    const int s0 = seq_of_row_fast(a, t0);
    strip = t0 - a.query_start_loc[s0] >= hist && t0 + R <= a.query_start_loc[s0 + 1];
  }
  if (R == 1 && hist <= kStripHist && a.width <= kNormThreads * kStripPerThread) {
    // a sequence's only row in this step (every row of a decode step; every row when there is no convolution): the row,
    // its predecessors from the carried state, and the state's shift, without a branch between the loads
    int q = 1, ctx = 0, slot = -1;
    if (hist > 0) {
      const int s = seq_of_row_fast(a, t0);
      q = a.query_start_loc[s + 1] - a.query_start_loc[s];
      ctx = a.context_lens[s];
      slot = a.slot_idx ? a.slot_idx[s] : -1;
    }
    if (q == 1) {
      elem* state = (hist > 0 && a.conv_state && slot >= 0) ? static_cast<elem*>(a.conv_state) + static_cast<int64_t>(slot) * hist * a.width
                                                            : nullptr;
      const bool carried = state != nullptr && ctx > 0;
      const float* row = a.x + static_cast<int64_t>(t0) * a.x_stride_t;
      float x[kStripPerThread], back[kStripHist][kStripPerThread];     // back[d - 1]: the normed row d steps back
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < kStripPerThread; ++u) {
        const int c = threadIdx.x + u * kNormThreads;
        x[u] = c < a.width ? row[c] : 0.f;
        ss = fmaf(x[u], x[u], ss);
#pragma unroll
        for (int d = 1; d <= kStripHist; ++d)
          back[d - 1][u] = (carried && d <= hist && c < a.width) ? A::ld(state + static_cast<int64_t>(hist - d) * a.width + c) : 0.f;
      }
      ss = wave_sum(ss);
      if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6][0] = ss;
      __syncthreads();
      float tot = 0.f;
#pragma unroll
      for (int w = 0; w < kNormWaves; ++w) tot += red[w][0];
      const float inv = 1.f / sqrtf(tot / static_cast<float>(a.width) + a.eps);
#pragma unroll
      for (int u = 0; u < kStripPerThread; ++u) {
        const int c = threadIdx.x + u * kNormThreads;
        if (c >= a.width) continue;
        const float n = A::round(x[u] * inv * (a.weight_offset + a.weight[c]));
        float acc = n;
        if (a.conv_weight != nullptr) {
          const float* cw = a.conv_weight + static_cast<int64_t>(c) * taps;
          acc = fmaf(cw[hist], n, acc);
#pragma unroll
          for (int d = kStripHist; d >= 1; --d)
            if (d <= hist) acc = fmaf(cw[hist - d], back[d - 1][u], acc);
        }
        A::st(static_cast<elem*>(a.out) + static_cast<int64_t>(t0) * a.width + c, acc);
        if (state != nullptr) {
          // the state moves up one row: the row d steps back goes to row hist - 1 - d, this row to the last
          A::st(state + static_cast<int64_t>(hist - 1) * a.width + c, n);
#pragma unroll
          for (int d = 1; d < kStripHist; ++d)
            if (d <= hist - 1) A::st(state + static_cast<int64_t>(hist - 1 - d) * a.width + c, back[d - 1][u]);
        }
      }
      return;
    }
  }
  if (!strip) {
    for (int r = 0; r < rows; ++r) {
      norm_conv_row<A>(a, t0 + r, red);
      __syncthreads();                         // red is reused by the next row
    }
    return;
  }
  // register image: input row t0 + R - 1 - m at v[m], m < R + hist (every index below is a compile-time constant)
  constexpr int kIn = R + kStripHist;
  float v[kIn][kStripPerThread];
  float ss[kIn];
#pragma unroll
  for (int m = 0; m < kIn; ++m) {
    ss[m] = 0.f;
    const bool used = m < R + hist;
    const float* row = a.x + (static_cast<int64_t>(t0) + R - 1 - m) * a.x_stride_t;
#pragma unroll
    for (int u = 0; u < kStripPerThread; ++u) {
      const int c = threadIdx.x + u * kNormThreads;
      v[m][u] = (used && c < a.width) ? row[c] : 0.f;
      ss[m] = fmaf(v[m][u], v[m][u], ss[m]);
    }
  }
#pragma unroll
  for (int m = 0; m < kIn; ++m) {
    const float w = wave_sum(ss[m]);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6][m] = w;
  }
  __syncthreads();
#pragma unroll
  for (int m = 0; m < kIn; ++m) {
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < kNormWaves; ++w) tot += red[w][m];
    const float inv = 1.f / sqrtf(tot / static_cast<float>(a.width) + a.eps);
#pragma unroll
    for (int u = 0; u < kStripPerThread; ++u) {
      const int c = threadIdx.x + u * kNormThreads;
      v[m][u] = c < a.width ? A::round(v[m][u] * inv * (a.weight_offset + a.weight[c])) : 0.f;
    }
  }
#pragma unroll
  for (int u = 0; u < kStripPerThread; ++u) {
    const int c = threadIdx.x + u * kNormThreads;
    if (c >= a.width) continue;
    float back[kStripHist + 1];                 // the tap that reads the row d steps back (d = 0: the row itself)
#pragma unroll
    for (int d = 0; d <= kStripHist; ++d) back[d] = d <= hist ? a.conv_weight[static_cast<int64_t>(c) * taps + hist - d] : 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float acc = v[R - 1 - r][u];
#pragma unroll
      for (int d = kStripHist; d >= 0; --d) acc = fmaf(back[d], v[R - 1 - r + d][u], acc);     // oldest row first, as the row form
      A::st(static_cast<elem*>(a.out) + (static_cast<int64_t>(t0) + r) * a.width + c, acc);
    }
  }
}

template <typename A>
__global__ __launch_bounds__(kNormThreads) void norm_residual_kernel(hymeta_norm_residual_args a) {
  typedef typename A::elem elem;
  __shared__ float red[kNormWaves];
  const int64_t t = blockIdx.x;
  const elem* y = static_cast<const elem*>(a.y) + t * a.y_stride_t;
  float* x = a.x + t * a.x_stride_t;
  float v[kMaxPerThread];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < kMaxPerThread; ++u) {
    const int c = threadIdx.x + u * kNormThreads;
    v[u] = c < a.width ? A::ld(y + c) : 0.f;
    ss += v[u] * v[u];
  }
  ss = block_sum<kNormWaves>(ss, red);
  const float inv = 1.f / sqrtf(ss / static_cast<float>(a.width) + a.eps);
#pragma unroll
  for (int u = 0; u < kMaxPerThread; ++u) {
    const int c = threadIdx.x + u * kNormThreads;
    if (c < a.width) {
      float r = x[c] + a.mult * (v[u] * inv * (a.weight_offset + a.weight[c]));
      if (a.post_add) r += a.post_add[c];
      x[c] = r;
    }
  }
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_embed_rows(const hymeta_embed_rows_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_embed_rows_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0 || a.vocab <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.token_ids || !a.table || !a.out) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(embed_rows_kernel<ActBf16>, dim3(a.num_tokens), dim3(kNormThreads), 0, st, a);
  else hipLaunchKernelGGL(embed_rows_kernel<ActF32>, dim3(a.num_tokens), dim3(kNormThreads), 0, st, a);
  return launch_status();
}

extern "C" int hymeta_norm_conv(const hymeta_norm_conv_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_norm_conv_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0 || a.num_seqs < 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.x || !a.weight || !a.out || a.x_stride_t < a.width) return HYMETA_ERR_INVALID_ARG;
  if (a.conv_weight) {
    if (a.taps < 1 || a.taps > HYMETA_CONV_MAX_TAPS) return HYMETA_ERR_UNSUPPORTED;
    if (a.taps > 1 && (a.num_seqs <= 0 || !a.query_start_loc || !a.context_lens)) return HYMETA_ERR_INVALID_ARG;
  }
  hipStream_t st = begin_launches(stream);
  // many rows: strips of four (their inputs read once); few rows (decode): a workgroup per row
  const bool strips = a.num_tokens >= 1024 && a.conv_weight != nullptr && a.taps > 1;
  const dim3 grid(strips ? (a.num_tokens + 3) / 4 : a.num_tokens);
  if (a.act_dtype == HYMETA_BF16) {
    if (strips) hipLaunchKernelGGL((norm_conv_kernel<ActBf16, 4>), grid, dim3(kNormThreads), 0, st, a);
    else hipLaunchKernelGGL((norm_conv_kernel<ActBf16, 1>), grid, dim3(kNormThreads), 0, st, a);
  } else {
    if (strips) hipLaunchKernelGGL((norm_conv_kernel<ActF32, 4>), grid, dim3(kNormThreads), 0, st, a);
    else hipLaunchKernelGGL((norm_conv_kernel<ActF32, 1>), grid, dim3(kNormThreads), 0, st, a);
  }
  return launch_status();
}

extern "C" int hymeta_norm_residual(const hymeta_norm_residual_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_norm_residual_args& a = *args;
  if (a.num_tokens < 0 || a.width <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.width > kNormThreads * kMaxPerThread) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.y || !a.weight || !a.x || a.x_stride_t < a.width || a.y_stride_t < a.width) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) hipLaunchKernelGGL(norm_residual_kernel<ActBf16>, dim3(a.num_tokens), dim3(kNormThreads), 0, st, a);
  else hipLaunchKernelGGL(norm_residual_kernel<ActF32>, dim3(a.num_tokens), dim3(kNormThreads), 0, st, a);
  return launch_status();
}
