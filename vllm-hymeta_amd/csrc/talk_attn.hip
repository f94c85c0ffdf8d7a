// Attention whose scores are mixed across heads before the softmax ("talking heads"), around its matrix products:
// the norms over the whole query / key projections, the rotation in interleaved pairs, the blend of the values with
// another layer's, the paged write, and the mix of the queries.
//
// score'_h(i, j) = sum_g talk[h, g] (q_g(i) . k_kv(g)(j)) is linear in the queries, so with the keys of a token's G
// key/value heads concatenated into one row K(j) it equals Q_h(i) . K(j), where Q_h(i)[kv D + d] = sum over the query heads
// g of group kv of talk[h, g] q_g(i)[d].  The attention itself is then hymeta_sink_attention with one shared key per
// token (HYMETA_KV_SHARED_KEY): no score ever leaves the attention kernel's registers to meet another head's.
#include "act_types.h"

namespace hymeta {

namespace {

constexpr int kMaxRotPairs = 512;
constexpr int kTalkLdsHeads = 64;      // the mix matrix of up to this many heads is read from LDS
constexpr int kGroupRegs = 16;         // query heads of a group a thread keeps in registers

__device__ __forceinline__ void store_pair(uint16_t* p, float a, float b) { *reinterpret_cast<uint32_t*>(p) = pack_bf16x2(a, b); }
__device__ __forceinline__ void store_pair(float* p, float a, float b) { *reinterpret_cast<u32x2*>(p) = u32x2{__float_as_uint(a), __float_as_uint(b)}; }

// grid = tokens; dynamic LDS: (H + G) * D floats (the normed and rotated queries and keys of the token).
// Vec: the row in fours of columns (aligned, H D and G D in whole fours) and the mixed queries in pairs (D even).
template <typename A, bool Vec>
__global__ __launch_bounds__(256) void talk_qkv_prep_kernel(hymeta_talk_qkv_prep_args a) {
  typedef typename A::elem elem;
  extern __shared__ __attribute__((aligned(16))) float s_qk[];
  __shared__ float s_cos[kMaxRotPairs], s_sin[kMaxRotPairs];
  __shared__ float red[4];
  __shared__ float s_talk[kTalkLdsHeads * kTalkLdsHeads];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int H = a.num_heads, G = a.num_kv_heads, D = a.head_dim, Dv = a.v_dim;
  const int nq = H * D, nk = G * D, nv = G * Dv, group = H / G;
  // what does not depend on the token goes first: the mix matrix is in LDS long before the mix reads it
  const float* talk = a.talk;
  if (H <= kTalkLdsHeads) {
    for (int i = tid; i < H * H; i += 256) s_talk[i] = a.talk[i];
    talk = s_talk;
  }
  int pos;
  if (a.positions) {
    pos = static_cast<int>(a.positions[t]);
  } else {
    const int s = seq_of_row(a.query_start_loc, a.num_seqs, t);
    pos = max(a.seq_lens[s] - (a.query_start_loc[s + 1] - t), 0);
  }
  const elem* row = static_cast<const elem*>(a.qkv) + static_cast<int64_t>(t) * a.qkv_stride_t;
  // angles in double precision, brought into [-pi, pi]; the functions are the fp32 ones on the remainder
  for (int i = tid; i < a.rot_dims / 2; i += 256) {
    constexpr double kTwoPi = 6.283185307179586476925286766559, kInvTwoPi = 0.15915494309189533576888376337251;
    const double ang = static_cast<double>(pos) * a.rot_freqs[i];
    const float r = static_cast<float>(fma(-kTwoPi, rint(ang * kInvTwoPi), ang));
    s_cos[i] = cosf(r);
    s_sin[i] = sinf(r);
  }
  float ssq = 0.f, ssk = 0.f;
  if (Vec) {
    for (int c = 4 * tid; c < nq + nk; c += 1024) {
      float v[4];
      A::ld4(row + c, v);
      *reinterpret_cast<f32x4*>(&s_qk[c]) = f32x4{v[0], v[1], v[2], v[3]};
      const float ss = (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
      if (c < nq) ssq += ss; else ssk += ss;
    }
  } else {
    for (int c = tid; c < nq + nk; c += 256) {
      const float v = A::ld(row + c);
      s_qk[c] = v;
      if (c < nq) ssq = fmaf(v, v, ssq); else ssk = fmaf(v, v, ssk);
    }
  }
  const float inv_q = 1.f / sqrtf(block_sum<4>(ssq, red) / static_cast<float>(nq) + a.eps);
  const float inv_k = 1.f / sqrtf(block_sum<4>(ssk, red) / static_cast<float>(nk) + a.eps);
  // norm and rotation in LDS: a thread takes a pair of the rotated dimensions, or one of the others
  for (int c = tid; c < nq + nk; c += 256) {
    const bool is_q = c < nq;
    const int d = (is_q ? c : c - nq) % D;
    const float* w = is_q ? a.q_weight : a.k_weight - nq;
    const float inv = is_q ? inv_q : inv_k;
    if (d < a.rot_dims) {
      if (d & 1) continue;
      const float u = s_qk[c] * inv * w[c], v = s_qk[c + 1] * inv * w[c + 1];
      const float cs = s_cos[d >> 1], sn = s_sin[d >> 1];
      s_qk[c] = u * cs - v * sn;
      s_qk[c + 1] = v * cs + u * sn;
    } else {
      s_qk[c] *= inv * w[c];
    }
  }
  __syncthreads();
  const int64_t slot = a.slot_mapping ? a.slot_mapping[t] : -1;
  if (a.kv_cache != nullptr && slot >= 0 && slot < a.num_blocks * a.block_size) {
    elem* dst = static_cast<elem*>(a.kv_cache) + slot * static_cast<int64_t>(nk + nv);
    for (int c = tid; c < nk; c += 256) A::st(dst + c, s_qk[nq + c]);
    const elem* v = row + nq + nk;
    const elem* vo = a.v_other ? static_cast<const elem*>(a.v_other) + static_cast<int64_t>(t) * a.v_other_stride_t : nullptr;
    for (int c = tid; c < nv; c += 256) {
      float r = A::ld(v + c);
      if (vo) r = (1.f - a.v_blend) * r + a.v_blend * A::ld(vo + c);
      A::st(dst + nk + c, r);
    }
  }
  // a thread takes columns of the shared key (a key/value head's dimension d; two neighbours in the Vec form) and walks
  // the query heads: the group's queries of those columns stay in registers, the mix weights are LDS broadcasts, the
  // stores of a wave are consecutive
  elem* qo = static_cast<elem*>(a.q_out) + static_cast<int64_t>(t) * H * nk;
  constexpr int kCols = Vec ? 2 : 1;
  for (int c = kCols * tid; c < nk; c += kCols * 256) {
    const int kv = c / D, d = c % D;
    const float* q = s_qk + (kv * group) * D + d;
    if (group <= kGroupRegs) {
      float qv[kGroupRegs][kCols];
#pragma unroll
      for (int j = 0; j < kGroupRegs; ++j)
#pragma unroll
        for (int e = 0; e < kCols; ++e) qv[j][e] = j < group ? q[j * D + e] : 0.f;
      for (int h = 0; h < H; ++h) {
        const float* tw = talk + h * H + kv * group;
        float r[kCols] = {};
#pragma unroll
        for (int j = 0; j < kGroupRegs; ++j)
          if (j < group) {
            const float wj = tw[j];
#pragma unroll
            for (int e = 0; e < kCols; ++e) r[e] = fmaf(wj, qv[j][e], r[e]);
          }
        if (Vec) store_pair(qo + static_cast<int64_t>(h) * nk + c, r[0], r[kCols - 1]);
        else A::st(qo + static_cast<int64_t>(h) * nk + c, r[0]);
      }
    } else {
      for (int h = 0; h < H; ++h) {
        const float* tw = talk + h * H + kv * group;
        float r[kCols] = {};
        for (int j = 0; j < group; ++j)
#pragma unroll
          for (int e = 0; e < kCols; ++e) r[e] = fmaf(tw[j], q[j * D + e], r[e]);
        if (Vec) store_pair(qo + static_cast<int64_t>(h) * nk + c, r[0], r[kCols - 1]);
        else A::st(qo + static_cast<int64_t>(h) * nk + c, r[0]);
      }
    }
  }
}

template <typename A>
void launch_talk_qkv_prep(const hymeta_talk_qkv_prep_args& a, size_t lds, hipStream_t st) {
  const int bytes = A::kDtype == HYMETA_BF16 ? 2 : 4;
  const bool vec = a.head_dim % 4 == 0 && reinterpret_cast<uintptr_t>(a.qkv) % (4 * bytes) == 0 && a.qkv_stride_t % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(a.q_out) % (2 * bytes) == 0;
  if (vec) {
    if (lds > 48 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(talk_qkv_prep_kernel<A, true>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    hipLaunchKernelGGL((talk_qkv_prep_kernel<A, true>), dim3(a.num_tokens), dim3(256), lds, st, a);
  } else {
    if (lds > 48 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(talk_qkv_prep_kernel<A, false>), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    hipLaunchKernelGGL((talk_qkv_prep_kernel<A, false>), dim3(a.num_tokens), dim3(256), lds, st, a);
  }
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_talk_qkv_prep(const hymeta_talk_qkv_prep_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_talk_qkv_prep_args& a = *args;
  if (a.num_tokens < 0 || a.num_seqs < 0 || a.num_heads <= 0 || a.num_kv_heads <= 0 || a.head_dim <= 0 || a.v_dim <= 0 || a.rot_dims < 0 ||
      a.block_size <= 0 || a.num_blocks < 0)
    return HYMETA_ERR_INVALID_ARG;
  if (a.num_heads % a.num_kv_heads != 0 || a.rot_dims % 2 != 0 || a.rot_dims > a.head_dim) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  const int64_t floats = static_cast<int64_t>(a.num_heads + a.num_kv_heads) * a.head_dim;
  if (a.rot_dims / 2 > kMaxRotPairs || floats * 4 > 96 * 1024) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_tokens == 0 || a.num_seqs == 0) return HYMETA_OK;
  if (!a.qkv || !a.q_weight || !a.k_weight || !a.talk || !a.q_out || (!a.positions && (!a.query_start_loc || !a.seq_lens)) || (a.rot_dims > 0 && !a.rot_freqs))
    return HYMETA_ERR_INVALID_ARG;
  if (a.slot_mapping && !a.kv_cache) return HYMETA_ERR_INVALID_ARG;
  if (a.qkv_stride_t < floats + static_cast<int64_t>(a.num_kv_heads) * a.v_dim) return HYMETA_ERR_INVALID_ARG;
  if (a.v_other && a.v_other_stride_t < static_cast<int64_t>(a.num_kv_heads) * a.v_dim) return HYMETA_ERR_INVALID_ARG;
  hipStream_t st = begin_launches(stream);
  const size_t lds = static_cast<size_t>(floats) * sizeof(float);
  if (a.act_dtype == HYMETA_BF16) launch_talk_qkv_prep<ActBf16>(a, lds, st);
  else launch_talk_qkv_prep<ActF32>(a, lds, st);
  return launch_status();
}
