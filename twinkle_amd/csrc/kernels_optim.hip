// Multi-tenant optimizer step: gradient normalisation, per-tenant gradient-norm clipping and AdamW for
// the adapter tensors of any number of tenants in three launches (two for the norms, one for the update),
// each tenant with its own token count, clip threshold and hyper-parameters.  Elementwise and HBM bound:
// one pass reads the gradients (norms), one pass reads parameter, gradient and both moments and writes
// parameter and moments.  Sums are formed in a fixed order (block tree, then blocks in index order per
// tenant), so the norms and with them the updates are bitwise repeatable.
#include <math.h>

#include "tk_device.h"

namespace tk {

namespace {

constexpr int kOptThreads = 256;
constexpr int kOptPerThread = 16;  // elements per thread
constexpr int kOptPerBlock = kOptThreads * kOptPerThread;

template <typename T>
__device__ inline float load_f32(const T* p, int64_t i) {
  return to_f32(p[i]);
}

// Block-wide reduction in a fixed order: sum or max of one float per thread, result in thread 0.
template <bool MAX>
__device__ inline float block_reduce(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    const float o = __shfl_xor(v, d, 64);
    v = MAX ? fmaxf(v, o) : v + o;
  }
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float r = scratch[0];
    for (int w = 1; w < kOptThreads / 64; ++w) r = MAX ? fmaxf(r, scratch[w]) : r + scratch[w];
    v = r;
  }
  return v;
}

// partial[tensor][block]: sum of squares (norm_type 2) or max of absolute values (norm_type inf) of the
// block's gradient elements, after division by the tenant's token count
template <typename T>
__global__ __launch_bounds__(kOptThreads) void k_opt_norm_partial(const tk_opt_tensor* __restrict__ tensors,
                                                                  const tk_opt_tenant* __restrict__ tenants,
                                                                  float* __restrict__ partial, int blocks_per_tensor) {
  __shared__ float scratch[kOptThreads / 64];
  const tk_opt_tensor t = tensors[blockIdx.y];
  const tk_opt_tenant h = tenants[t.tenant];
  const int64_t i0 = (int64_t)blockIdx.x * kOptPerBlock;
  if (!h.active || i0 >= t.numel) return;  // the final pass reads only the blocks a tensor really has
  const bool inf = isinf(h.norm_type);
  const T* g = (const T*)t.grad;
  float acc = 0.f;
  constexpr int V = 16 / sizeof(T);  // elements per 16-byte load
  const int64_t i1 = min(i0 + kOptPerBlock, t.numel);
  if ((reinterpret_cast<uintptr_t>(g) & 15u) == 0 && ((i1 - i0) % V) == 0) {
    // 16-byte loads, consecutive threads on consecutive pieces
    for (int64_t i = i0 + (int64_t)threadIdx.x * V; i < i1; i += (int64_t)kOptThreads * V) {
      const uint4 raw = *reinterpret_cast<const uint4*>(g + i);
      float v[8];
      if (sizeof(T) == 2) {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          v[2 * k] = __uint_as_float(w[k] << 16);
          v[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
        }
      } else {
        v[0] = __uint_as_float(raw.x); v[1] = __uint_as_float(raw.y);
        v[2] = __uint_as_float(raw.z); v[3] = __uint_as_float(raw.w);
      }
#pragma unroll
      for (int k = 0; k < V; ++k) {
        const float x = v[k] * h.grad_scale;
        acc = inf ? fmaxf(acc, fabsf(x)) : acc + x * x;
      }
    }
  } else {
    for (int64_t i = i0 + threadIdx.x; i < i1; i += kOptThreads) {
      const float x = load_f32(g, i) * h.grad_scale;
      acc = inf ? fmaxf(acc, fabsf(x)) : acc + x * x;
    }
  }
  acc = inf ? block_reduce<true>(acc, scratch) : block_reduce<false>(acc, scratch);
  if (threadIdx.x == 0) partial[(int64_t)blockIdx.y * blocks_per_tensor + blockIdx.x] = acc;
}

// One block per tenant: every thread adds the partials of a fixed share of the tenant's tensors in a fixed
// order, then the block tree.  norm[tenant] = total norm after normalisation, before clipping;
// clip[tenant] = min(1, max_grad_norm / (norm + 1e-6)) (torch.nn.utils.clip_grad_norm_'s coefficient).
__global__ __launch_bounds__(kOptThreads) void k_opt_norm_final(const tk_opt_tensor* __restrict__ tensors, int n_tensors,
                                                                const tk_opt_tenant* __restrict__ tenants,
                                                                const float* __restrict__ partial, int blocks_per_tensor,
                                                                float* __restrict__ norm_out,
                                                                float* __restrict__ clip_out) {
  __shared__ float scratch[kOptThreads / 64];
  const int tenant = blockIdx.x;
  const tk_opt_tenant h = tenants[tenant];
  if (!h.active) {
    if (threadIdx.x == 0) {
      norm_out[tenant] = 0.f;
      clip_out[tenant] = 1.f;
    }
    return;
  }
  const bool inf = isinf(h.norm_type);
  float acc = 0.f;
  // a thread takes every 256th tensor and adds that tensor's blocks in block order
  for (int ti = threadIdx.x; ti < n_tensors; ti += kOptThreads) {
    if (tensors[ti].tenant != tenant) continue;
    const int nb = (int)((tensors[ti].numel + kOptPerBlock - 1) / kOptPerBlock);
    const float* p = partial + (int64_t)ti * blocks_per_tensor;
    for (int b = 0; b < nb; ++b) acc = inf ? fmaxf(acc, p[b]) : acc + p[b];
  }
  acc = inf ? block_reduce<true>(acc, scratch) : block_reduce<false>(acc, scratch);
  if (threadIdx.x == 0) {
    const float norm = inf ? acc : sqrtf(acc);
    norm_out[tenant] = norm;
    clip_out[tenant] = h.max_grad_norm > 0.f ? fminf(1.f, h.max_grad_norm / (norm + 1e-6f)) : 1.f;
  }
}

// AdamW with decoupled weight decay, fp32 arithmetic, fp32 moments (torch.optim.AdamW without amsgrad /
// maximize): g' = g * grad_scale * clip;  p *= 1 - lr wd;  m = m + (1 - b1)(g' - m);  v = b2 v + (1 - b2) g'^2;
// p -= lr / (1 - b1^t) * m / (sqrt(v) / sqrt(1 - b2^t) + eps).
template <typename T>
__global__ __launch_bounds__(kOptThreads) void k_opt_adamw(const tk_opt_tensor* __restrict__ tensors,
                                                           const tk_opt_tenant* __restrict__ tenants,
                                                           const float* __restrict__ clip, int flags) {
  const tk_opt_tensor t = tensors[blockIdx.y];
  const tk_opt_tenant h = tenants[t.tenant];
  const int64_t i0 = (int64_t)blockIdx.x * kOptPerBlock;
  if (!h.active || i0 >= t.numel) return;
  const float gs = h.grad_scale * (clip ? clip[t.tenant] : 1.f);
  const float bc2_sqrt = h.bias_correction2_sqrt;
  const float step_size = h.lr / h.bias_correction1;
  const float decay = 1.f - h.lr * h.weight_decay;
  T* p = (T*)t.param;
  T* g = (T*)t.grad;
#pragma unroll 4
  for (int j = 0; j < kOptPerThread; ++j) {
    const int64_t i = i0 + (int64_t)j * kOptThreads + threadIdx.x;
    if (i >= t.numel) break;
    const float gv = load_f32(g, i) * gs;
    float pv = load_f32(p, i) * decay;
    float m = t.exp_avg[i], v = t.exp_avg_sq[i];
    m = m + h.one_minus_beta1 * (gv - m);
    v = h.beta2 * v + h.one_minus_beta2 * gv * gv;
    pv -= step_size * (m / (sqrtf(v) / bc2_sqrt + h.eps));
    t.exp_avg[i] = m;
    t.exp_avg_sq[i] = v;
    from_f32(pv, &p[i]);
    if (flags & TK_OPT_ZERO_GRADS) from_f32(0.f, &g[i]);
    else if (flags & TK_OPT_WRITE_GRADS) from_f32(gv, &g[i]);
  }
}

}  // namespace

int launch_opt_grad_norm(const tk_opt_tensor* tensors, int n_tensors, const tk_opt_tenant* tenants, int n_tenants,
                         int64_t max_numel, int dtype, float* norm_out, float* clip_out, float* partial,
                         hipStream_t s) {
  const int bpt = (int)ceil_div(max_numel, kOptPerBlock);
  const dim3 grid((unsigned)bpt, (unsigned)n_tensors);
  if (n_tensors > 0 && dtype == TK_DTYPE_F32)
    hipLaunchKernelGGL(k_opt_norm_partial<float>, grid, dim3(kOptThreads), 0, s, tensors, tenants, partial, bpt);
  else if (n_tensors > 0)
    hipLaunchKernelGGL(k_opt_norm_partial<bf16_t>, grid, dim3(kOptThreads), 0, s, tensors, tenants, partial, bpt);
  hipLaunchKernelGGL(k_opt_norm_final, dim3((unsigned)n_tenants), dim3(kOptThreads), 0, s, tensors, n_tensors, tenants,
                     partial, bpt, norm_out, clip_out);
  return check_launch();
}

int launch_opt_adamw(const tk_opt_tensor* tensors, int n_tensors, const tk_opt_tenant* tenants, int64_t max_numel,
                     int dtype, const float* clip, int flags, hipStream_t s) {
  const dim3 grid((unsigned)ceil_div(max_numel, kOptPerBlock), (unsigned)n_tensors);
  if (dtype == TK_DTYPE_F32)
    hipLaunchKernelGGL(k_opt_adamw<float>, grid, dim3(kOptThreads), 0, s, tensors, tenants, clip, flags);
  else
    hipLaunchKernelGGL(k_opt_adamw<bf16_t>, grid, dim3(kOptThreads), 0, s, tensors, tenants, clip, flags);
  return check_launch();
}

int64_t opt_partial_floats(int n_tensors, int64_t max_numel) {
  return (int64_t)n_tensors * ceil_div(max_numel, kOptPerBlock);
}

}  // namespace tk
