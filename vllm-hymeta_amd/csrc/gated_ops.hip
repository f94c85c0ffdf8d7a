// Elementwise activations between two projections: the clamped gated unit of the experts, xIELU of the dense
// feed-forward, an output gate, the silu-gated unit and the squared relu.  act_dtype in and out, fp32 inside.
#include "act_types.h"

namespace hymeta {

namespace {

__device__ __forceinline__ float clamped_glu(float gate, float up, float limit, float alpha) {
  const float g = fminf(gate, limit);
  const float u = fminf(fmaxf(up, -limit), limit);
  return g * sigmoid_exact(alpha * g) * (u + 1.f);
}

__device__ __forceinline__ float xielu(float z, float a_pos, float a_neg) {
  return z > 0.f ? fmaf(a_pos * z, z, 0.5f * z) : fmaf(a_neg, expm1f(z) - z, 0.5f * z);
}

__device__ __forceinline__ float apply(int kind, float v0, float v1, float p0, float p1) {
  if (kind == HYMETA_ACT_CLAMPED_GLU) return clamped_glu(v0, v1, p0, p1);
  if (kind == HYMETA_ACT_XIELU) return xielu(v0, p0, p1);
  if (kind == HYMETA_ACT_SILU_MUL) return v0 * sigmoid_exact(v0) * v1;
  if (kind == HYMETA_ACT_RELU2) return fmaxf(v0, 0.f) * fmaxf(v0, 0.f);
  return v0 * sigmoid_exact(v1);
}

// grid = (rows, runs of 1024 columns): a thread takes four columns of a row -- consecutive ones with one load and one
// store each where the pointers and strides are in whole fours (Vec), else the columns tid, tid + 256, ...
template <typename A, int Kind, bool Vec>
__global__ __launch_bounds__(256) void activation_kernel(hymeta_activation_args a) {
  typedef typename A::elem elem;
  const int rows = a.num_rows_dev ? min(*a.num_rows_dev, a.num_rows) : a.num_rows;
  const int c0 = blockIdx.y * 1024;
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const elem* x = static_cast<const elem*>(a.x) + r * a.x_stride;
    const elem* second = (Kind == HYMETA_ACT_CLAMPED_GLU || Kind == HYMETA_ACT_SILU_MUL) ? x + a.n : Kind == HYMETA_ACT_SIGMOID_MUL ? static_cast<const elem*>(a.gate) + r * a.gate_stride : nullptr;
    elem* out = static_cast<elem*>(a.out) + r * a.out_stride;
    float v0[4], v1[4] = {}, v[4];
    if (Vec) {
      const int c = c0 + 4 * threadIdx.x;
      if (c >= a.n) continue;
      A::ld4(x + c, v0);
      if (Kind != HYMETA_ACT_XIELU && Kind != HYMETA_ACT_RELU2) A::ld4(second + c, v1);
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = apply(Kind, v0[u], v1[u], a.p0, a.p1);
      A::st4(out + c, v);
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + threadIdx.x + 256 * u;
        v0[u] = c < a.n ? A::ld(x + c) : 0.f;
        if (Kind != HYMETA_ACT_XIELU && Kind != HYMETA_ACT_RELU2) v1[u] = c < a.n ? A::ld(second + c) : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + threadIdx.x + 256 * u;
        if (c < a.n) A::st(out + c, apply(Kind, v0[u], v1[u], a.p0, a.p1));
      }
    }
  }
}

template <typename A, int Kind>
void launch_activation(const hymeta_activation_args& a, hipStream_t st) {
  const int bytes = A::kDtype == HYMETA_BF16 ? 2 : 4;
  auto fours = [&](const void* p, int64_t stride) { return p == nullptr || (reinterpret_cast<uintptr_t>(p) % (4 * bytes) == 0 && stride % 4 == 0); };
  const bool vec = a.n % 4 == 0 && fours(a.x, a.x_stride) && fours(a.out, a.out_stride) && (Kind != HYMETA_ACT_SIGMOID_MUL || fours(a.gate, a.gate_stride));
  const dim3 grid(a.num_rows < 65535 ? a.num_rows : 65535, (a.n + 1023) / 1024);
  if (vec) hipLaunchKernelGGL((activation_kernel<A, Kind, true>), grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL((activation_kernel<A, Kind, false>), grid, dim3(256), 0, st, a);
}

template <typename A>
void launch_activation_kind(const hymeta_activation_args& a, hipStream_t st) {
  if (a.kind == HYMETA_ACT_CLAMPED_GLU) launch_activation<A, HYMETA_ACT_CLAMPED_GLU>(a, st);
  else if (a.kind == HYMETA_ACT_XIELU) launch_activation<A, HYMETA_ACT_XIELU>(a, st);
  else if (a.kind == HYMETA_ACT_SILU_MUL) launch_activation<A, HYMETA_ACT_SILU_MUL>(a, st);
  else if (a.kind == HYMETA_ACT_RELU2) launch_activation<A, HYMETA_ACT_RELU2>(a, st);
  else launch_activation<A, HYMETA_ACT_SIGMOID_MUL>(a, st);
}

}  // namespace

}  // namespace hymeta

using namespace hymeta;

extern "C" int hymeta_activation(const hymeta_activation_args* args, hymeta_stream_t stream) {
  if (!args_ok(args)) return HYMETA_ERR_INVALID_ARG;
  const hymeta_activation_args& a = *args;
  if (a.num_rows < 0 || a.n <= 0) return HYMETA_ERR_INVALID_ARG;
  if (!act_dtype_ok(a.act_dtype)) return HYMETA_ERR_UNSUPPORTED;
  if (a.kind < HYMETA_ACT_CLAMPED_GLU || a.kind > HYMETA_ACT_RELU2) return HYMETA_ERR_UNSUPPORTED;
  if (a.num_rows == 0) return HYMETA_OK;
  if (!a.x || !a.out || (a.kind == HYMETA_ACT_SIGMOID_MUL && !a.gate)) return HYMETA_ERR_INVALID_ARG;
  const int64_t in_cols = (a.kind == HYMETA_ACT_CLAMPED_GLU || a.kind == HYMETA_ACT_SILU_MUL) ? 2 * static_cast<int64_t>(a.n) : a.n;
  if (a.x_stride < in_cols || a.out_stride < a.n || (a.kind == HYMETA_ACT_SIGMOID_MUL && a.gate_stride < a.n)) return HYMETA_ERR_INVALID_ARG;
  if ((a.n + 1023) / 1024 > 65535) return HYMETA_ERR_UNSUPPORTED;
  hipStream_t st = begin_launches(stream);
  if (a.act_dtype == HYMETA_BF16) launch_activation_kind<ActBf16>(a, st);
  else launch_activation_kind<ActF32>(a, st);
  return launch_status();
}
