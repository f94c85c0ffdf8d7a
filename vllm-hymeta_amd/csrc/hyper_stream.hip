// Several fp32 residual streams per token ("hyper-connections") and their start:
//   embed_pair    token embedding + hashed (previous, current) pair embedding, layer norm, copied into every stream
//   hyper_stream  spread a sublayer's output over a remix of the streams and/or read the next sublayer's input as a
//                 layer norm of a weighted sum of the streams, one launch
// Everything is fp32 but the tables, the sublayer's output and the normed rows handed to the next projection.
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kPer = 32;            // columns a thread keeps (width <= 256 * kPer)

// (x - mean) / sqrt(var + eps) of a row spread over the workgroup as v[u] = column tid + 256 u; var = mean of the
// squared deviations (two passes over the registers).
__device__ __forceinline__ void row_layer_norm(float* v, int width, float eps, float* red) {
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < kPer; ++u) s += v[u];               // (columns past the width hold zero)
  const float mean = block_sum<4>(s, red) / static_cast<float>(width);
  float q = 0.f;
#pragma unroll
  for (int u = 0; u < kPer; ++u) {
    const int c = threadIdx.x + 256 * u;
    const float d = c < width ? v[u] - mean : 0.f;
    v[u] = d;
    q = fmaf(d, d, q);
  }
  const float inv = 1.f / sqrtf(block_sum<4>(q, red) / static_cast<float>(width) + eps);
#pragma unroll
  for (int u = 0; u < kPer; ++u) v[u] *= inv;
}

__device__ __forceinline__ int64_t pair_row(int64_t prev, int64_t cur, const hymeta_embed_pair_args& a) {
  return (prev * a.mul_prev + cur * a.mul_cur) % a.buckets;
}

// a thread per sequence: the pair row of the portion's first token (from the state), then the state's new value
__global__ __launch_bounds__(64) void pair_first_rows_kernel(hymeta_embed_pair_args a) {
  const int s = blockIdx.x * 64 + threadIdx.x;
  if (s >= a.num_seqs) return;
  const int lo = a.query_start_loc[s], hi = a.query_start_loc[s + 1];
  if (hi <= lo) return;
  const int slot = a.slot_idx ? a.slot_idx[s] : -1;
  const bool carried = a.context_lens[s] > 0 && slot >= 0;
  a.first_rows[s] = carried ? static_cast<int32_t>(pair_row(a.prev_token[slot], a.token_ids[lo], a)) : static_cast<int32_t>(a.buckets);
  if (slot >= 0) a.prev_token[slot] = static_cast<int32_t>(a.token_ids[hi - 1]);
}

// grid = tokens
template <typename A>
__global__ __launch_bounds__(256) void embed_pair_kernel(hymeta_embed_pair_args a) {
  typedef typename A::elem elem;
  __shared__ float red[4];
  const int t = blockIdx.x, W = a.width;
  const int64_t tok = a.token_ids[t];
  const elem* e = static_cast<const elem*>(a.table) + (tok >= 0 && tok < a.vocab ? tok : 0) * W;
  const elem* p = nullptr;
  if (a.pair_table) {
    const int s = seq_of_row(a.query_start_loc, a.num_seqs, t);
    const int64_t row = t == a.query_start_loc[s] ? a.first_rows[s] : pair_row(a.token_ids[t - 1], tok, a);
    p = static_cast<const elem*>(a.pair_table) + row * W;
  }
  float v[kPer];
#pragma unroll
  for (int u = 0; u < kPer; ++u) {
    const int c = threadIdx.x + 256 * u;
    v[u] = c < W ? A::ld(e + c) + (p ? A::ld(p + c) : 0.f) : 0.f;
  }
  if (a.norm_weight) row_layer_norm(v, W, a.eps, red);
  float* out = a.out + static_cast<int64_t>(t) * a.copies * W;
#pragma unroll
  for (int u = 0; u < kPer; ++u) {
    const int c = threadIdx.x + 256 * u;
    if (c < W) {
      const float r = a.norm_weight ? v[u] * a.norm_weight[c] : v[u];
      for (int k = 0; k < a.copies; ++k) out[static_cast<int64_t>(k) * W + c] = r;
    }
  }
}

// Layer norm of a row held as NV groups of four consecutive columns per thread (group u = columns 4 (tid + 256 u) ..).
template <int NV>
__device__ __forceinline__ void row_layer_norm4(float (&v)[NV][4], int width, float eps, float* red) {
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < NV; ++u) s += (v[u][0] + v[u][1]) + (v[u][2] + v[u][3]);        // (groups past the width hold zero)
  const float mean = block_sum<4>(s, red) / static_cast<float>(width);
  float q = 0.f;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const bool in = 4 * (static_cast<int>(threadIdx.x) + 256 * u) < width;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float d = in ? v[u][e] - mean : 0.f;
      v[u][e] = d;
      q = fmaf(d, d, q);
    }
  }
  const float inv = 1.f / sqrtf(block_sum<4>(q, red) / static_cast<float>(width) + eps);
#pragma unroll
  for (int u = 0; u < NV; ++u)
#pragma unroll
    for (int e = 0; e < 4; ++e) v[u][e] *= inv;
}

// grid = tokens; the row in NV groups of four consecutive columns per thread (width in whole fours, aligned tables)
template <typename A, int NV>
__global__ __launch_bounds__(256) void embed_pair4_kernel(hymeta_embed_pair_args a) {
  typedef typename A::elem elem;
  __shared__ float red[4];
  const int t = blockIdx.x, W = a.width;
  const int64_t tok = a.token_ids[t];
  const elem* e = static_cast<const elem*>(a.table) + (tok >= 0 && tok < a.vocab ? tok : 0) * W;
  const elem* p = nullptr;
  if (a.pair_table) {
    const int s = seq_of_row(a.query_start_loc, a.num_seqs, t);
    const int64_t row = t == a.query_start_loc[s] ? a.first_rows[s] : pair_row(a.token_ids[t - 1], tok, a);
    p = static_cast<const elem*>(a.pair_table) + row * W;
  }
  float v[NV][4];
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int c = 4 * (threadIdx.x + 256 * u);
#pragma unroll
    for (int k = 0; k < 4; ++k) v[u][k] = 0.f;
    if (c < W) {
      A::ld4(e + c, v[u]);
      if (p) {
        float pv[4];
        A::ld4(p + c, pv);
#pragma unroll
        for (int k = 0; k < 4; ++k) v[u][k] += pv[k];
      }
    }
  }
  if (a.norm_weight) row_layer_norm4<NV>(v, W, a.eps, red);
  float* out = a.out + static_cast<int64_t>(t) * a.copies * W;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int c = 4 * (threadIdx.x + 256 * u);
    if (c < W) {
      if (a.norm_weight) {
        float wv[4];
        ActF32::ld4(a.norm_weight + c, wv);
#pragma unroll
        for (int k = 0; k < 4; ++k) v[u][k] *= wv[k];
      }
      for (int k = 0; k < a.copies; ++k) ActF32::st4(out + static_cast<int64_t>(k) * W + c, v[u]);
    }
  }
}

template <typename A>
void launch_embed_pair(const hymeta_embed_pair_args& a, hipStream_t st) {
  const int bytes = A::kDtype == HYMETA_BF16 ? 2 : 4;
  auto aligned = [&](const void* p, int b) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % (4 * b) == 0; };
  const dim3 grid(a.num_tokens), block(256);
  if (a.width % 4 != 0 || !aligned(a.table, bytes) || !aligned(a.pair_table, bytes) || !aligned(a.out, 4) || !aligned(a.norm_weight, 4)) {
    hipLaunchKernelGGL(embed_pair_kernel<A>, grid, block, 0, st, a);
    return;
  }
  const int groups = (a.width / 4 + 255) / 256;
  if (groups <= 1) hipLaunchKernelGGL((embed_pair4_kernel<A, 1>), grid, block, 0, st, a);
  else if (groups <= 2) hipLaunchKernelGGL((embed_pair4_kernel<A, 2>), grid, block, 0, st, a);
  else if (groups <= 4) hipLaunchKernelGGL((embed_pair4_kernel<A, 4>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((embed_pair4_kernel<A, 8>), grid, block, 0, st, a);
}

// grid = tokens.  S: streams, NV: groups of four columns a thread takes (both compile time, so that a column's streams and
// the row stay in registers); width in whole fours, 16-byte loads and stores of the fp32 streams.
template <typename A, int S, int NV>
__global__ __launch_bounds__(256) void hyper_stream_kernel(hymeta_hyper_stream_args a) {
  typedef typename A::elem elem;
  __shared__ float red[4];
  __shared__ float s_mix[S * S], s_out[S], s_in[S];
  const int t = blockIdx.x, W = a.width;
  if (threadIdx.x < S * S) s_mix[threadIdx.x] = a.y ? a.mix[threadIdx.x] : 0.f;
  if (threadIdx.x < S) {
    s_out[threadIdx.x] = a.y ? a.out_w[threadIdx.x] : 0.f;
    s_in[threadIdx.x] = a.h_out ? a.in_w[threadIdx.x] : 0.f;
  }
  __syncthreads();
  float* x = a.x + static_cast<int64_t>(t) * S * W;
  const elem* y = a.y ? static_cast<const elem*>(a.y) + static_cast<int64_t>(t) * a.y_stride_t : nullptr;
  float v[NV][4];
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int c = 4 * (threadIdx.x + 256 * u);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[u][e] = 0.f;
    if (c < W) {
      float xs[S][4];
#pragma unroll
      for (int s = 0; s < S; ++s) ActF32::ld4(x + s * W + c, xs[s]);
      if (y) {
        float yv[4], nx[S][4];
        A::ld4(y + c, yv);
#pragma unroll
        for (int to = 0; to < S; ++to)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float r = s_out[to] * yv[e];
#pragma unroll
            for (int from = 0; from < S; ++from) r = fmaf(s_mix[from * S + to], xs[from][e], r);
            nx[to][e] = r;
          }
#pragma unroll
        for (int s = 0; s < S; ++s) {
#pragma unroll
          for (int e = 0; e < 4; ++e) xs[s][e] = nx[s][e];
          ActF32::st4(x + s * W + c, nx[s]);
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float r = 0.f;
#pragma unroll
        for (int s = 0; s < S; ++s) r = fmaf(s_in[s], xs[s][e], r);
        v[u][e] = r;
      }
    }
  }
  if (!a.h_out) return;
  if (a.norm_weight) row_layer_norm4<NV>(v, W, a.eps, red);
  elem* h = static_cast<elem*>(a.h_out) + static_cast<int64_t>(t) * W;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int c = 4 * (threadIdx.x + 256 * u);
    if (c < W) {
      if (a.norm_weight) {
        float wv[4];
        ActF32::ld4(a.norm_weight + c, wv);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[u][e] *= wv[e];
      }
      A::st4(h + c, v[u]);
    }
  }
}

// Any width, more than 8 streams, pointers that are not 16-byte aligned: a column per thread and round, the weighted sum through LDS
// (dynamic: width floats) between the rounds.
template <typename A>
__global__ __launch_bounds__(256) void hyper_stream_any_kernel(hymeta_hyper_stream_args a) {
  typedef typename A::elem elem;
  extern __shared__ float s_u[];
  __shared__ float red[4];
  const int t = blockIdx.x, W = a.width, S = a.streams;
  float* x = a.x + static_cast<int64_t>(t) * S * W;
  const elem* y = a.y ? static_cast<const elem*>(a.y) + static_cast<int64_t>(t) * a.y_stride_t : nullptr;
  float sum = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    float xs[HYMETA_MAX_STREAMS], nx[HYMETA_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < HYMETA_MAX_STREAMS; ++s) xs[s] = s < S ? x[s * W + c] : 0.f;
    if (y) {
      const float yv = A::ld(y + c);
#pragma unroll
      for (int to = 0; to < HYMETA_MAX_STREAMS; ++to) {
        float r = 0.f;
        if (to < S) {
          r = a.out_w[to] * yv;
#pragma unroll
          for (int from = 0; from < HYMETA_MAX_STREAMS; ++from)
            if (from < S) r = fmaf(a.mix[from * S + to], xs[from], r);
          x[to * W + c] = r;
        }
        nx[to] = r;
      }
#pragma unroll
      for (int s = 0; s < HYMETA_MAX_STREAMS; ++s) xs[s] = nx[s];
    }
    if (a.h_out) {
      float r = 0.f;
#pragma unroll
      for (int s = 0; s < HYMETA_MAX_STREAMS; ++s)
        if (s < S) r = fmaf(a.in_w[s], xs[s], r);
      s_u[c] = r;
      sum += r;
    }
  }
  if (!a.h_out) return;
  elem* h = static_cast<elem*>(a.h_out) + static_cast<int64_t>(t) * W;
  float mean = 0.f, inv = 1.f;
  if (a.norm_weight) {
    mean = block_sum<4>(sum, red) / static_cast<float>(W);
    float q = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) q = fmaf(s_u[c] - mean, s_u[c] - mean, q);      // (a thread reads what it wrote)
    inv = 1.f / sqrtf(block_sum<4>(q, red) / static_cast<float>(W) + a.eps);
  }
  for (int c = threadIdx.x; c < W; c += 256) A::st(h + c, a.norm_weight ? (s_u[c] - mean) * inv * a.norm_weight[c] : s_u[c]);
}

template <typename A, int S>
void launch_hyper_stream_s(const hymeta_hyper_stream_args& a, hipStream_t st) {
  const dim3 grid(a.num_tokens), block(256);
  const int groups = (a.width / 4 + 255) / 256;
  if (groups <= 1) hipLaunchKernelGGL((hyper_stream_kernel<A, S, 1>), grid, block, 0, st, a);
  else if (groups <= 2) hipLaunchKernelGGL((hyper_stream_kernel<A, S, 2>), grid, block, 0, st, a);
  else if (groups <= 4) hipLaunchKernelGGL((hyper_stream_kernel<A, S, 4>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((hyper_stream_kernel<A, S, 8>), grid, block, 0, st, a);
}

template <typename A>
void launch_hyper_stream(const hymeta_hyper_stream_args& a, hipStream_t st) {
  const int bytes = A::kDtype == HYMETA_BF16 ? 2 : 4;
  auto fours = [&](const void* p, int64_t stride, int b) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) % (4 * b) == 0 && stride % 4 == 0); };
  const bool vec = a.width % 4 == 0 && fours(a.x, a.width, 4) && fours(a.y, a.y_stride_t, bytes) && fours(a.h_out, a.width, bytes) &&
                   fours(a.norm_weight, 4, 4);
  if (!vec || a.streams > 8) {
    hipLaunchKernelGGL(hyper_stream_any_kernel<A>, dim3(a.num_tokens), dim3(256), a.h_out ? a.width * sizeof(float) : 0, st, a);
    return;
  }
  switch (a.streams) {
    case 1: launch_hyper_stream_s<A, 1>(a, st); break;
    case 2: launch_hyper_stream_s<A, 2>(a, st); break;
    case 3: launch_hyper_stream_s<A, 3>(a, st); break;
    case 4: launch_hyper_stream_s<A, 4>(a, st); break;
    case 5: launch_hyper_stream_s<A, 5>(a, st); break;
    case 6: launch_hyper_stream_s<A, 6>(a, st); break;
    case 7: launch_hyper_stream_s<A, 7>(a, st); break;
    default: launch_hyper_stream_s<A, 8>(a, st); break;
  }
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_embed_pair(const hymeta_embed_pair_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_embed_pair_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.width <= 0 || a.vocab <= 0 || a.copies <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.width > 256 * kPer) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.token_ids || !a.table || !a.out) return HYMETA_ERR_INVALID_ARG;
  if (a.pair_table && (a.buckets <= 0 || a.mul_prev < 0 || a.mul_cur < 0 || a.num_seqs <= 0 || !a.query_start_loc || !a.context_lens || !a.first_rows ||
                       (a.slot_idx && !a.prev_token)))
    return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.pair_table) hipLaunchKernelGGL(pair_first_rows_kernel, dim3((a.num_seqs + 63) / 64), dim3(64), 0, st, a);
  if (a.act_dtype == HYMETA_BF16) launch_embed_pair<ActBf16>(a, st);
  else launch_embed_pair<ActF32>(a, st);
  return launch_status();
}

extern "C" int hymeta_hyper_stream(const hymeta_hyper_stream_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_hyper_stream_args& a = *args;
  if (a.num_tokens < 0 || a.streams <= 0 || a.width <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.streams > HYMETA_MAX_STREAMS || a.width > 256 * kPer) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0) return HYMETA_OK;
  if (!a.x || (!a.y && !a.h_out)) return HYMETA_ERR_INVALID_ARG;
  if (a.y && (!a.mix || !a.out_w || a.y_stride_t < a.width)) return HYMETA_ERR_INVALID_ARG;
  if (a.h_out && !a.in_w) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) launch_hyper_stream<ActBf16>(a, st);
  else launch_hyper_stream<ActF32>(a, st);
  return launch_status();
}
