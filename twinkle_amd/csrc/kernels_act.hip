// Gated activation between the two expert projections: hidden = silu(gate) * up with gate | up side by side in
// one row of the gate_up output, and its backward.  Elementwise and HBM-bound: every thread moves 8 consecutive
// columns (16 bytes in bf16) of gate, up and the result; the arithmetic is done in fp32 and rounded once.
// As separate torch kernels (silu, mul, their backward, the concatenation of the two gradients) the same work
// crosses memory about three times as often.
#include "tk_device.h"

namespace tk {

namespace {

template <typename T>
struct alignas(8 * sizeof(T)) Vec8 {
  T v[8];
};

template <typename T>
__device__ inline void load8(const T* p, float (&f)[8]) {
  const Vec8<T> x = *reinterpret_cast<const Vec8<T>*>(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = to_f32(x.v[i]);
}
template <typename T>
__device__ inline void store8(T* p, const float (&f)[8]) {
  Vec8<T> x;
#pragma unroll
  for (int i = 0; i < 8; ++i) from_f32(f[i], &x.v[i]);
  *reinterpret_cast<Vec8<T>*>(p) = x;
}

__device__ inline float sigmoidf(float x) { return 1.f / (1.f + __expf(-x)); }

template <typename T>
__global__ __launch_bounds__(256) void k_swiglu_fwd(const T* __restrict__ gu, int64_t ld_in, T* __restrict__ out,
                                                    int64_t ld_out, int64_t rows, int inter) {
  const int per_row = inter >> 3;
  const int64_t total = rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / per_row;
    const int c = (int)(i - r * per_row) << 3;
    float g[8], u[8], o[8];
    load8(gu + r * ld_in + c, g);
    load8(gu + r * ld_in + inter + c, u);
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = g[k] * sigmoidf(g[k]) * u[k];
    store8(out + r * ld_out + c, o);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void k_swiglu_bwd(const T* __restrict__ gu, int64_t ld_in,
                                                    const T* __restrict__ dout, int64_t ld_dout,
                                                    T* __restrict__ dgu, int64_t ld_dgu, int64_t rows, int inter) {
  const int per_row = inter >> 3;
  const int64_t total = rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / per_row;
    const int c = (int)(i - r * per_row) << 3;
    float g[8], u[8], d[8], dg[8], du[8];
    load8(gu + r * ld_in + c, g);
    load8(gu + r * ld_in + inter + c, u);
    load8(dout + r * ld_dout + c, d);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float s = sigmoidf(g[k]);
      du[k] = d[k] * g[k] * s;                                // d/d up   = silu(gate)
      dg[k] = d[k] * u[k] * s * (1.f + g[k] * (1.f - s));     // d/d gate = up * silu'(gate)
    }
    store8(dgu + r * ld_dgu + c, dg);
    store8(dgu + r * ld_dgu + inter + c, du);
  }
}

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

}  // namespace

int launch_swiglu(const void* gu, int64_t ld_in, const void* dout, int64_t ld_dout, void* out, int64_t ld_out,
                  int64_t rows, int inter, int dtype, hipStream_t s) {
  if (rows == 0) return TK_OK;
  const size_t vec = dtype == TK_DTYPE_BF16 ? 16 : 32;
  if (inter % 8 != 0 || ld_in % 8 != 0 || ld_out % 8 != 0 || (dout && ld_dout % 8 != 0) || !aligned_to(gu, vec) ||
      !aligned_to(out, vec) || (dout && !aligned_to(dout, vec)))
    return TK_ERR_UNSUPPORTED;
  const int64_t total = rows * (inter >> 3);
  const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div(total, 256), 256 * 32);
  if (dtype == TK_DTYPE_BF16) {
    if (dout)
      hipLaunchKernelGGL(k_swiglu_bwd<bf16_t>, dim3(blocks), dim3(256), 0, s, (const bf16_t*)gu, ld_in,
                         (const bf16_t*)dout, ld_dout, (bf16_t*)out, ld_out, rows, inter);
    else
      hipLaunchKernelGGL(k_swiglu_fwd<bf16_t>, dim3(blocks), dim3(256), 0, s, (const bf16_t*)gu, ld_in, (bf16_t*)out,
                         ld_out, rows, inter);
  } else {
    if (dout)
      hipLaunchKernelGGL(k_swiglu_bwd<float>, dim3(blocks), dim3(256), 0, s, (const float*)gu, ld_in,
                         (const float*)dout, ld_dout, (float*)out, ld_out, rows, inter);
    else
      hipLaunchKernelGGL(k_swiglu_fwd<float>, dim3(blocks), dim3(256), 0, s, (const float*)gu, ld_in, (float*)out,
                         ld_out, rows, inter);
  }
  return check_launch();
}

}  // namespace tk
