// Device helpers shared by the bf16 MFMA kernel files (gfx950).
//
// MFMA operand layout of v_mfma_f32_16x16x32_bf16 (l = lane, 64 lanes):
//   A operand: lane l holds A[i = l % 16][k = 8 * (l / 16) .. + 8]   (8 bf16 = 16 B)
//   B operand: lane l holds B[k = 8 * (l / 16) .. + 8][j = l % 16]
//   D        : lane l holds D[i = 4 * (l / 16) + v][j = l % 16], v = 0..3
#pragma once

#include "tk_device.h"

namespace tk {

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

__device__ inline f32x4 mfma16(uint4 a, uint4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                 0, 0);
}

__device__ inline uint4 ld16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ inline void st16(bf16_t* p, uint4 v) { *reinterpret_cast<uint4*>(p) = v; }
// Streaming (non-temporal) variants for data that is touched exactly once per pass.  The expand
// kernel's read-modify-write of y / dx uses them: marked this way its 256 MB do not linger as dirty
// lines in L2 and in the last-level cache, and the kernels that follow it run up to 20 % faster (the
// whole step 8 %).  On the read-only streams of the other kernels they made no difference.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ inline uint4 ld16_nt(const bf16_t* p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ inline void st16_nt(bf16_t* p, uint4 v) {
  const u32x4_t w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<u32x4_t*>(p));
}
__device__ inline uint4 zero4() { return make_uint4(0u, 0u, 0u, 0u); }

// two floats -> packed bf16 pair (round to nearest even; one v_cvt_pk_bf16_f32 on gfx950)
__device__ inline uint32_t pack_bf16(float lo, float hi) {
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
  typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
  f32x2 f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}
__device__ inline float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ inline float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// Block barrier that orders LDS traffic only: unlike __syncthreads() it does not wait for the global
// loads a wave has in flight, so software-pipelined loads stay outstanding across it.
__device__ inline void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// keep the first `keep` (0..8) bf16 elements of a quad, zero the rest
__device__ inline uint4 keep_first(uint4 v, int keep) {
  if (keep >= 8) return v;
  if (keep <= 0) return zero4();
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int e = keep - 2 * d;  // elements of this dword that stay
    w[d] = e >= 2 ? w[d] : (e == 1 ? (w[d] & 0xffffu) : 0u);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}
// Eight consecutive bf16 results: one 16-byte store when `vec`, element stores otherwise; `keep` (1..8)
// elements are written, the rest of the destination is left alone.
__device__ inline void store_bf16x8(bf16_t* o, const float (&v)[8], int keep, bool accumulate, bool vec) {
  if (vec && keep >= 8) {
    float f[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = v[i];
    if (accumulate) {
      const uint4 old = ld16(o);
      f[0] += bf16_lo(old.x); f[1] += bf16_hi(old.x); f[2] += bf16_lo(old.y); f[3] += bf16_hi(old.y);
      f[4] += bf16_lo(old.z); f[5] += bf16_hi(old.z); f[6] += bf16_lo(old.w); f[7] += bf16_hi(old.w);
    }
    st16(o, make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7])));
    return;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if (i >= keep) break;
    float val = v[i];
    if (accumulate) val += to_f32(o[i]);
    o[i] = (bf16_t)(pack_bf16(val, 0.f) & 0xffffu);
  }
}

// The same into an fp32 gradient: two 16-byte stores when `vec` (destination 16-byte aligned).
__device__ inline void store_f32x8(float* o, const float (&v)[8], int keep, bool accumulate, bool vec) {
  if (vec && keep >= 8) {
    float4 lo = make_float4(v[0], v[1], v[2], v[3]), hi = make_float4(v[4], v[5], v[6], v[7]);
    if (accumulate) {
      const float4 a = *reinterpret_cast<const float4*>(o), b = *reinterpret_cast<const float4*>(o + 4);
      lo.x += a.x; lo.y += a.y; lo.z += a.z; lo.w += a.w;
      hi.x += b.x; hi.y += b.y; hi.z += b.z; hi.w += b.w;
    }
    *reinterpret_cast<float4*>(o) = lo;
    *reinterpret_cast<float4*>(o + 4) = hi;
    return;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if (i >= keep) break;
    o[i] = accumulate ? o[i] + v[i] : v[i];
  }
}

// Blocks go to the XCDs (each with an L2 of its own) round-robin.  This renumbering gives every XCD one
// contiguous eighth of the work items, so that an XCD's L2 fetches the weights of few groups instead of all.
__device__ inline int xcd_contiguous(int block, int blocks) {
  const int per = blocks >> 3;
  return block < 8 * per ? (block & 7) * per + (block >> 3) : block;
}

// One wave's weight-gradient block out[n][c0 .. c0 + 127] (lane holds out[16 nb + li][32 kb + 8 v + q] in
// acc[q][nb][v]) leaves through `lds` (RP rows of kWgradStageStride floats, private to the wave) as whole
// 512-byte rows: into the chunk's slot of the partial buffer, or straight into the gradient when the
// chunk is its group's only one.
constexpr int kWgradStageStride = 132;  // 4 mod 32: conflict-free 16-byte accesses
template <int NB>
__device__ inline void wgrad_store(const f32x4 (&acc)[8][NB], float* lds, const WgradArgs& a, const ChunkInfo& ci,
                                   int g, int r_all, int c0, int lane, int n_base = 0) {
  const int r = r_all - n_base;  // live rows of this block of 16 NB rank indices, which starts at n_base
  constexpr int RP = 16 * NB, OS = kWgradStageStride;
  const int li = lane & 15, kb = lane >> 4;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      float* o = lds + (16 * nb + li) * OS + 32 * kb + 8 * v;
      *reinterpret_cast<float4*>(o) = make_float4(acc[0][nb][v], acc[1][nb][v], acc[2][nb][v], acc[3][nb][v]);
      *reinterpret_cast<float4*>(o + 4) = make_float4(acc[4][nb][v], acc[5][nb][v], acc[6][nb][v], acc[7][nb][v]);
    }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");

  if (ci.partial >= 0) {
    float* part = a.partial + partial_index(ci.partial, n_base, c0, a.rpad, a.width);  // c0 is a multiple of 128
#pragma unroll
    for (int i = 0; i < RP / 2; ++i) {
      const int n = 2 * i + (lane >> 5), c = 4 * (lane & 31);
      if (n < r) *reinterpret_cast<float4*>(part + n * 128 + c) = *reinterpret_cast<const float4*>(lds + n * OS + c);
    }
    return;
  }
  if (a.grad_f32) {  // fp32 gradients next to bf16 activations: the same two walks with fp32 stores
    float* gf = (float*)a.grad[g];
    const bool vecf = (reinterpret_cast<uintptr_t>(gf) & 15u) == 0 && (a.ld_grad & 3) == 0;
    if (!a.transposed) {
#pragma unroll
      for (int i = 0; i < RP / 4; ++i) {
        const int n = 4 * i + kb, c = 8 * li;
        if (n >= r) continue;
        const float4 lo = *reinterpret_cast<const float4*>(lds + n * OS + c);
        const float4 hi = *reinterpret_cast<const float4*>(lds + n * OS + c + 4);
        const float v8[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        store_f32x8(gf + (int64_t)(n_base + n) * a.ld_grad + c0 + c, v8, 8, a.accumulate != 0, vecf);
      }
    } else {
      // grad[c0 + c][n]: neighbouring lanes take neighbouring rank octets of one column, so that a wave-wide store
      // covers runs of whole rows of the gradient instead of one 16-byte (32-byte) piece of each of 64 rows
#pragma unroll
      for (int k = 0; k < RP / 4; ++k) {
        const int piece = lane + 64 * k, c = piece / (RP / 8), n8 = 8 * (piece % (RP / 8));
        if (n8 >= r) continue;
        float v8[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v8[i] = lds[(n8 + i) * OS + c];
        store_f32x8(gf + (int64_t)(c0 + c) * a.ld_grad + n_base + n8, v8, min(8, r - n8), a.accumulate != 0, vecf);
      }
    }
    return;
  }
  bf16_t* gp = (bf16_t*)a.grad[g];
  const bool vec = (reinterpret_cast<uintptr_t>(gp) & 15u) == 0 && (a.ld_grad & 7) == 0;
  if (!a.transposed) {
    // grad[n][c0 + c]: four rows of 128 columns per step
#pragma unroll
    for (int i = 0; i < RP / 4; ++i) {
      const int n = 4 * i + kb, c = 8 * li;
      if (n >= r) continue;
      const float4 lo = *reinterpret_cast<const float4*>(lds + n * OS + c);
      const float4 hi = *reinterpret_cast<const float4*>(lds + n * OS + c + 4);
      const float v8[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      store_bf16x8(gp + (int64_t)(n_base + n) * a.ld_grad + c0 + c, v8, 8, a.accumulate != 0, vec);
    }
  } else {
    // grad[c0 + c][n]: neighbouring lanes take neighbouring rank octets of one column (see above)
#pragma unroll
    for (int k = 0; k < RP / 4; ++k) {
      const int piece = lane + 64 * k, c = piece / (RP / 8), n8 = 8 * (piece % (RP / 8));
      if (n8 >= r) continue;
      float v8[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) v8[i] = lds[(n8 + i) * OS + c];
      store_bf16x8(gp + (int64_t)(c0 + c) * a.ld_grad + n_base + n8, v8, min(8, r - n8), a.accumulate != 0, vec);
    }
  }
}

}  // namespace

}  // namespace tk
