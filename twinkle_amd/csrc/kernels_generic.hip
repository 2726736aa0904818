// Shape-agnostic kernels for the segmented LoRA pass: fp32 or bf16 storage,
// fp32 accumulation on the vector ALUs, any width / stride / rank <= 128.
// They carry the fp32 configuration and every shape the MFMA kernels do not
// take (odd widths, unaligned strides), and share all buffers and tables with
// them, so the two families are interchangeable per launch.
#include <algorithm>

#include "tk_device.h"

namespace tk {

namespace {

constexpr int kKC = 64;   // source columns staged per step in the shrink kernel

// hT[n][slot] = scale_g * sum_k src[row(slot)][k] * W_g[n][k]   for the 32 slots of one tile
template <typename T>
__global__ __launch_bounds__(256) void k_shrink_generic(PassArgs a, const int32_t* __restrict__ tile_group,
                                                        const int32_t* __restrict__ slot_rows) {
  extern __shared__ float lds_f[];
  const int tile_id = blockIdx.x;
  const int g = checked_group(tile_group[tile_id], a.tb);
  if (g < 0) return;
  const int r = class_rank(a.rank[g], a.rank_lo, a.rpad);
  if (a.class_mode && r <= 0) return;  // a group of another rank class: its tiles belong to another launch
  const int rpad = a.rpad;
  float* xs = lds_f;                          // [32][kKC + 1]
  float* ws = lds_f + kTileRows * (kKC + 1);  // [rpad][kKC + 1]
  __shared__ int rows_s[kTileRows];
  const int tid = threadIdx.x;
  const int slot0 = tile_id * kTileRows;
  if (tid < kTileRows) rows_s[tid] = checked_row(slot_rows[slot0 + tid], a.tb);
  __syncthreads();
  const T* src = (const T*)a.src;
  const T* W = group_weight<T>(a.w_shrink, a.w_shrink_base, a.shrink_group_stride, g);
  const int row = tid & 31;   // tile row this thread accumulates
  const int ng = tid >> 5;    // rank indices ng, ng + 8, ...
  float acc[TK_MAX_RANK / 8];
#pragma unroll
  for (int j = 0; j < TK_MAX_RANK / 8; ++j) acc[j] = 0.f;
  const int nacc = (rpad + 7) / 8;
  for (int k0 = 0; k0 < a.width_src; k0 += kKC) {
    for (int i = tid; i < kTileRows * kKC; i += 256) {
      const int rr = i / kKC, kk = i % kKC;
      const int k = k0 + kk;
      xs[rr * (kKC + 1) + kk] =
          (k < a.width_src && rows_s[rr] >= 0) ? to_f32(src[(int64_t)rows_s[rr] * a.ld_src + k]) : 0.f;
    }
    for (int i = tid; i < rpad * kKC; i += 256) {
      const int n = i / kKC, kk = i % kKC;
      const int k = k0 + kk;
      ws[n * (kKC + 1) + kk] = (n < r && k < a.width_src) ? to_f32(W[(int64_t)n * a.ld_shrink + k]) : 0.f;
    }
    __syncthreads();
    for (int kk = 0; kk < kKC; ++kk) {
      const float xv = xs[row * (kKC + 1) + kk];
#pragma unroll
      for (int j = 0; j < TK_MAX_RANK / 8; ++j)
        if (j < nacc) acc[j] += xv * ws[(ng + 8 * j) * (kKC + 1) + kk];
    }
    __syncthreads();
  }
  const float sc = r > 0 ? a.scale[g] : 0.f;
  T* hT = (T*)a.hT;
  T* hrow = hT + (int64_t)rpad * a.ldh;
  // padding slots hold exact zeros so that the row-contraction kernels need no masks
#pragma unroll
  for (int j = 0; j < TK_MAX_RANK / 8; ++j) {
    const int n = ng + 8 * j;
    if (n < rpad) {
      T hv;
      from_f32((n < r && rows_s[row] >= 0) ? acc[j] * sc : 0.f, &hv);
      hT[(int64_t)n * a.ldh + slot0 + row] = hv;
      hrow[(int64_t)(slot0 + row) * rpad + n] = hv;
    }
  }
}

// dst[row(slot)][c] += sum_n hT[n][slot] * W_g[c][n]   for the 32 slots of one tile
template <typename T>
__global__ __launch_bounds__(256) void k_expand_generic(PassArgs a, const int32_t* __restrict__ tile_group,
                                                        const int32_t* __restrict__ slot_rows) {
  extern __shared__ float lds_f[];  // hs[rpad][32]
  const int tile_id = blockIdx.x;
  const int g = checked_group(tile_group[tile_id], a.tb);
  if (g < 0) return;
  const int r = class_rank(a.rank[g], a.rank_lo, a.rpad);
  if (r <= 0) return;
  __shared__ int rows_s[kTileRows];
  const int tid = threadIdx.x;
  const int slot0 = tile_id * kTileRows;
  if (tid < kTileRows) rows_s[tid] = checked_row(slot_rows[slot0 + tid], a.tb);
  const T* hT = (const T*)a.hT;
  for (int i = tid; i < r * kTileRows; i += 256) {
    const int n = i / kTileRows, rr = i % kTileRows;
    lds_f[i] = to_f32(hT[(int64_t)n * a.ldh + slot0 + rr]);
  }
  __syncthreads();
  const T* W = group_weight<T>(a.w_expand, a.w_expand_base, a.expand_group_stride, g);
  T* dst = (T*)a.dst;
  for (int c = tid; c < a.width_dst; c += 256) {
    float acc[kTileRows];
#pragma unroll
    for (int rr = 0; rr < kTileRows; ++rr) acc[rr] = 0.f;
    const T* wrow = W + (int64_t)c * a.ld_expand;
    for (int n = 0; n < r; ++n) {
      const float b = to_f32(wrow[n]);
#pragma unroll
      for (int rr = 0; rr < kTileRows; ++rr) acc[rr] += lds_f[n * kTileRows + rr] * b;
    }
#pragma unroll
    for (int rr = 0; rr < kTileRows; ++rr) {
      if (rows_s[rr] >= 0) {
        T* o = dst + (int64_t)rows_s[rr] * a.ld_dst + c;
        from_f32(to_f32(*o) + acc[rr], o);
      }
    }
  }
}

template <typename T>
__device__ inline void store_grad(const WgradArgs& a, int g, int n, int c, float v) {
  if (sizeof(T) != 4 && a.grad_f32) {  // fp32 gradient next to bf16 activations
    store_grad<float>(a, g, n, c, v);
    return;
  }
  T* gp = (T*)a.grad[g];
  T* o = a.transposed ? gp + (int64_t)c * a.ld_grad + n : gp + (int64_t)n * a.ld_grad + c;
  if (a.accumulate) v += to_f32(*o);
  from_f32(v, o);
}

// One chunk of one group, 256 columns per block, walked in passes of 512 slots:
// out[n][c] = sum_{slot in chunk} hT[n][slot] * src[row(slot)][c], slots ascending.
template <typename T>
__global__ __launch_bounds__(256) void k_wgrad_generic(WgradArgs a, const ChunkInfo* __restrict__ chunks,
                                                       const int32_t* __restrict__ slot_rows) {
  constexpr int kPass = kChunkTilesMin * kTileRows;
  __shared__ float hs[16][kPass];
  __shared__ int rows_s[kPass];
  const ChunkInfo ci = checked_chunk(chunks[blockIdx.x], a.tb);
  const int g = ci.group;
  if (g < 0) return;
  const int r = class_rank(a.rank[g], a.rank_lo, a.rpad);
  if (r <= 0) return;
  const int tid = threadIdx.x;
  const int c = blockIdx.y * 256 + tid;
  const int total = ci.ntiles * kTileRows;
  const T* src = (const T*)a.src;
  const T* hT = (const T*)a.hT;
  for (int n0 = 0; n0 < r; n0 += 16) {
    float acc[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = 0.f;
    for (int p0 = 0; p0 < total; p0 += kPass) {
      const int slot0 = ci.tile0 * kTileRows + p0;
      const int len = min(kPass, total - p0);
      __syncthreads();
      for (int i = tid; i < len; i += 256) rows_s[i] = checked_row(slot_rows[slot0 + i], a.tb);
      for (int i = tid; i < 16 * len; i += 256) {
        const int j = i / len, pp = i % len;
        hs[j][pp] = (n0 + j) < r ? to_f32(hT[(int64_t)(n0 + j) * a.ldh + slot0 + pp]) : 0.f;
      }
      __syncthreads();
      if (c < a.width) {
        for (int pp = 0; pp < len; ++pp) {
          if (rows_s[pp] < 0) continue;
          const float xv = to_f32(src[(int64_t)rows_s[pp] * a.ld_src + c]);
#pragma unroll
          for (int j = 0; j < 16; ++j) acc[j] += hs[j][pp] * xv;
        }
      }
    }
    if (c < a.width) {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int n = n0 + j;
        if (n < r) {
          if (ci.partial >= 0)
            a.partial[partial_index(ci.partial, n, c, a.rpad, a.width)] = acc[j];
          else
            store_grad<T>(a, g, n, c, acc[j]);
        }
      }
    }
  }
}

// Groups with several chunks: sum their partials in chunk order.  Groups with
// no rows: clear the live block when overwriting.  One (group, 8 rank
// indices, 256 columns) per block, a thread owns one column of the eight, so
// that a transposed gradient ([width][r], dB) leaves as 16-byte pieces instead
// of single elements; blockIdx.z >= rpad / 8 selects the second argument set,
// so that the reductions of dA and dB share one launch.
// PAIRED: chunks were taken in pairs (WgradArgs::pair_chunks), so only some slots hold sums.  A compile-time switch:
// the kernel's time is the chain from its first loads to its stores, and the slot arithmetic in that chain cost the
// unpaired launch 1 us of its 10.
template <typename T, bool PAIRED>
__device__ __forceinline__ void wgrad_reduce_body(const WgradArgs& a, int n0, const int32_t* __restrict__ chunk_first,
                                                  const int32_t* __restrict__ partial_first) {
  if (a.grad == nullptr) return;
  const int g = blockIdx.x;
  // independent loads first
  const int rk = a.rank[g], cf0 = chunk_first[g], cf1 = chunk_first[g + 1], pf = partial_first[g];
  const int r = class_rank(rk, a.rank_lo, a.rpad);
  const int nchunk = cf1 - cf0;
  // (table entries are compared with the table's bounds before they index: see TableBounds)
  if (nchunk < 0 || (nchunk > 1 && (pf < 0 || pf > a.tb.max_partials - nchunk))) return;
  if (nchunk == 1) return;
  if (nchunk == 0 && a.accumulate) return;
  // paired chunks (WgradArgs::pair_chunks): only every other slot behind the first holds a sum
  const int nlive = PAIRED && nchunk > 0 ? live_partials(nchunk, pf) : nchunk;  // (no chunks: zeros are written)
  auto slot = [&](int m) { return PAIRED ? live_partial(m, pf) : m; };
  const int64_t stride = partial_slot_floats(a.rpad, a.width);
  T* const gt = (T*)a.grad[g];
  if (a.transposed && (a.ld_grad & (sizeof(T) == 2 ? 7 : 3)) == 0 && (reinterpret_cast<uintptr_t>(gt) & 15u) == 0 &&
      (r & 7) == 0) {
    // A transposed gradient ([width][r], dB) whose rows are whole 16-byte pieces.  With a thread per column and an
    // octet of rank indices per block every 128-byte line of it was written in up to eight partial stores from eight
    // blocks (measured at 14336 columns, rank 64: 40 of the kernel's 79 us).  Here a block owns all octets of its
    // columns: it reads the partial sums with neighbouring threads on neighbouring columns (whole lines of the
    // partial buffer), turns the sums over in LDS and writes with neighbouring threads on neighbouring octets,
    // i.e. whole rows of the gradient.  The blocks of a group are renumbered: block (y, octet z) takes the columns
    // [b cpb, b cpb + cpb), b = y * (rpad / 8) + z, cpb = 256 / octets per column.
    __shared__ __attribute__((aligned(16))) float turn[256 * 8];
    if (r == 0) return;
    int noct = 1;
    while (8 * noct < r) noct <<= 1;  // octets per column, padded to a power of two
    const int cpb = 256 / noct, tid = threadIdx.x;
    const int col0 = (blockIdx.y * (a.rpad >> 3) + (n0 >> 3)) * cpb;
    if (col0 >= a.width) return;  // (block-uniform, like every return above)
    {
      const int oct = tid / cpb, cl = tid % cpb, c = col0 + cl;
      float acc[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = 0.f;
      if (c < a.width && 8 * oct < r) {
        const float* p = a.partial + partial_index(pf, 8 * oct, c, a.rpad, a.width);
        for (int j0 = 0; j0 < nlive; j0 += 2) {
          float v[2][8];
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < 8; ++i) v[j][i] = j0 + j < nlive ? p[slot(j0 + j) * stride + i * 128] : 0.f;
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] += v[j][i];
        }
      }
      float4* o = reinterpret_cast<float4*>(turn + (cl * noct + oct) * 8);
      o[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
      o[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
    }
    __syncthreads();
    const int oct = tid & (noct - 1), c = col0 + tid / noct;
    if (c >= a.width || 8 * oct >= r) return;
    const float4 lo = *reinterpret_cast<const float4*>(turn + tid * 8), hi = *reinterpret_cast<const float4*>(turn + tid * 8 + 4);
    float acc[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    if constexpr (sizeof(T) == 4) {  // fp32 gradient: the octet is two 16-byte pieces
      float4* of = reinterpret_cast<float4*>(gt + (int64_t)c * a.ld_grad + 8 * oct);
      if (a.accumulate) {
        const float4 o0 = of[0], o1 = of[1];
        acc[0] += o0.x; acc[1] += o0.y; acc[2] += o0.z; acc[3] += o0.w;
        acc[4] += o1.x; acc[5] += o1.y; acc[6] += o1.z; acc[7] += o1.w;
      }
      of[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
      of[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
      return;
    }
    uint4* o = reinterpret_cast<uint4*>(gt + (int64_t)c * a.ld_grad + 8 * oct);
    if (a.accumulate) {
      const uint4 old = *o;
      const uint32_t w[4] = {old.x, old.y, old.z, old.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[2 * i] += __uint_as_float(w[i] << 16);
        acc[2 * i + 1] += __uint_as_float(w[i] & 0xffff0000u);
      }
    }
    uint16_t h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) from_f32(acc[i], &h[i]);
    *o = make_uint4(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16), h[4] | ((uint32_t)h[5] << 16),
                    h[6] | ((uint32_t)h[7] << 16));
    return;
  }
  if (n0 >= r) return;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= a.width) return;
  const float* p = a.partial + partial_index(pf, n0, c, a.rpad, a.width);
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  // two chunks (16 loads) are requested together; every sum adds its chunks in chunk order
  for (int j0 = 0; j0 < nlive; j0 += 2) {
    float v[2][8];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < 8; ++i)
        v[j][i] = (j0 + j < nlive && n0 + i < r) ? p[slot(j0 + j) * stride + i * 128] : 0.f;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += v[j][i];
  }
  T* gp = (T*)a.grad[g];
  if (sizeof(T) == 2 && a.transposed && n0 + 8 <= r && (a.ld_grad & 7) == 0 &&
      (reinterpret_cast<uintptr_t>(gp) & 15u) == 0) {
    uint4* o = reinterpret_cast<uint4*>(gp + (int64_t)c * a.ld_grad + n0);
    if (a.accumulate) {
      const uint4 old = *o;
      const uint32_t w[4] = {old.x, old.y, old.z, old.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[2 * i] += __uint_as_float(w[i] << 16);
        acc[2 * i + 1] += __uint_as_float(w[i] & 0xffff0000u);
      }
    }
    uint16_t h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) from_f32(acc[i], &h[i]);
    *o = make_uint4(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16), h[4] | ((uint32_t)h[5] << 16),
                    h[6] | ((uint32_t)h[7] << 16));
    return;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i)
    if (n0 + i < r) store_grad<T>(a, g, n0 + i, c, acc[i]);
}

template <typename T>
__global__ __launch_bounds__(256) void k_wgrad_reduce(WgradArgs a0, WgradArgs a1, int rpad,
                                                      const int32_t* __restrict__ chunk_first,
                                                      const int32_t* __restrict__ partial_first) {
  const int zsets = rpad >> 3;
  const bool second = (int)blockIdx.z >= zsets;
  const WgradArgs& a = second ? a1 : a0;
  const int n0 = 8 * (second ? blockIdx.z - zsets : blockIdx.z);
  if (a.pair_chunks) wgrad_reduce_body<T, true>(a, n0, chunk_first, partial_first);
  else wgrad_reduce_body<T, false>(a, n0, chunk_first, partial_first);
}

// Any number of argument sets of one padded rank (dA and dB of several projections) in one launch:
// blockIdx.z = octets * set + octet of rank indices, octets = rpad / 8.
template <typename T>
__global__ __launch_bounds__(256) void k_wgrad_reduce_multi(WgradReduceJobs jobs, int octets,
                                                            const int32_t* __restrict__ chunk_first,
                                                            const int32_t* __restrict__ partial_first) {
  const int set = blockIdx.z / octets;
  const WgradArgs& a = jobs.a[set];
  const int n0 = 8 * (blockIdx.z - set * octets);
  if (a.pair_chunks) wgrad_reduce_body<T, true>(a, n0, chunk_first, partial_first);
  else wgrad_reduce_body<T, false>(a, n0, chunk_first, partial_first);
}

// bT_g[n][m] = B_g[m][n], aT_g[k][n] = A_g[n][k]; zero for n >= rank[g].
// (TS: the adapters' element type, T: that of the copies; they differ for fp32 adapters under bf16 activations)
template <typename TS, typename T>
__global__ __launch_bounds__(256) void k_transpose_weights(tk_lora_desc d, int rpad, int rank_lo, T* __restrict__ bT,
                                                           T* __restrict__ aT) {
  const int g = blockIdx.y;
  const int r = class_rank(d.rank[g], rank_lo, rpad);
  if (rank_lo > 0 && r <= 0) return;  // a group of a lower rank class: no launch of this class reads its copies
  const TS* A = (const TS*)d.lora_A[g];
  const TS* B = (const TS*)d.lora_B[g];
  const int64_t nb = (int64_t)rpad * d.out_features, na = (int64_t)rpad * d.in_features;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nb + na; i += (int64_t)gridDim.x * 256) {
    if (i < nb) {
      const int n = (int)(i / d.out_features), m = (int)(i % d.out_features);
      T v = (T)0;
      if (n < r) from_f32(to_f32(B[(int64_t)m * d.ldb + n]), &v);
      bT[(int64_t)g * nb + i] = v;
    } else {
      const int64_t q = i - nb;
      const int k = (int)(q / rpad), n = (int)(q % rpad);
      T v = (T)0;
      if (n < r) from_f32(to_f32(A[(int64_t)n * d.lda + k]), &v);
      aT[(int64_t)g * na + q] = v;
    }
  }
}

// bf16 copies of fp32 adapter weights (see WeightStage): the live rows of A_g as [rpad][in_features], the live
// columns of B_g as [out_features][rpad], eight elements per thread, and the two pointer tables.  Round to
// nearest even, as a cast of the tensors would.
struct ConvertJobs {  // one job per projection (blockIdx.z); a single call has one
  tk_lora_desc d[kMaxShared];
  char* stage[kMaxShared];
  WeightStage W[kMaxShared];
  int32_t rpad[kMaxShared];
};

__global__ __launch_bounds__(256) void k_convert_weights(ConvertJobs jobs, int want_a, int want_b) {
  const tk_lora_desc& d = jobs.d[blockIdx.z];
  const WeightStage& W = jobs.W[blockIdx.z];
  char* stage = jobs.stage[blockIdx.z];
  const int rpad = jobs.rpad[blockIdx.z];
  const int g = blockIdx.y;
  if (g >= d.num_groups) return;
  bf16_t* ac = (bf16_t*)(stage + W.off_a) + (int64_t)g * W.stride_a;
  bf16_t* bc = (bf16_t*)(stage + W.off_b) + (int64_t)g * W.stride_b;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (want_a) ((const void**)(stage + W.off_ptr_a))[g] = ac;
    if (want_b) ((const void**)(stage + W.off_ptr_b))[g] = bc;
  }
  const int r = min(d.rank[g], rpad);
  const float* A = (const float*)d.lora_A[g];
  const float* B = (const float*)d.lora_B[g];
  const int k8 = (d.in_features + 7) >> 3, n8 = rpad >> 3;
  const bool vec_a = (d.lda & 3) == 0 && (reinterpret_cast<uintptr_t>(A) & 15u) == 0;
  const bool vec_b = (d.ldb & 3) == 0 && (reinterpret_cast<uintptr_t>(B) & 15u) == 0;
  const int64_t units_a = want_a ? (int64_t)r * k8 : 0;                 // (n, k-octet)
  const int64_t units_b = want_b ? (int64_t)d.out_features * n8 : 0;    // (m, n-octet)
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < units_a + units_b; u += (int64_t)gridDim.x * 256) {
    float v[8];
    bf16_t* o;
    int keep;
    if (u < units_a) {
      const int n = (int)(u / k8), k0 = (int)(u % k8) * 8;
      keep = min(8, d.in_features - k0);
      const float* src = A + (int64_t)n * d.lda + k0;
      if (vec_a && keep == 8) {
        const float4 lo = *reinterpret_cast<const float4*>(src), hi = *reinterpret_cast<const float4*>(src + 4);
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = j < keep ? src[j] : 0.f;
      }
      o = ac + (int64_t)n * d.in_features + k0;
    } else {
      const int64_t q = u - units_a;
      const int m = (int)(q / n8), n0 = (int)(q % n8) * 8;
      keep = 8;  // the copy's rows are rpad long: columns past the rank are written as zeros
      const float* src = B + (int64_t)m * d.ldb + n0;
      if (vec_b && n0 + 8 <= r) {
        const float4 lo = *reinterpret_cast<const float4*>(src), hi = *reinterpret_cast<const float4*>(src + 4);
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = n0 + j < r ? src[j] : 0.f;
      }
      o = bc + (int64_t)m * rpad + n0;
    }
    if (keep == 8 && (reinterpret_cast<uintptr_t>(o) & 15u) == 0) {  // one 16-byte store
      uint16_t h[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) from_f32(v[j], &h[j]);
      *reinterpret_cast<uint4*>(o) = make_uint4(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16),
                                                h[4] | ((uint32_t)h[5] << 16), h[6] | ((uint32_t)h[7] << 16));
      continue;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < keep) from_f32(v[j], &o[j]);
  }
}

}  // namespace

int launch_convert_weights_multi(const tk_lora_desc* const* d, void* const* stage, int n, bool want_a, bool want_b,
                                 hipStream_t s) {
  if (n < 1 || n > kMaxShared) return TK_ERR_INVALID;
  ConvertJobs J{};
  int64_t per_group = 0;
  int groups = 0;
  for (int p = 0; p < n; ++p) {
    const int rpad = rank_pad(d[p]->max_rank);
    J.d[p] = *d[p];
    J.stage[p] = (char*)stage[p];
    J.W[p] = WeightStage(d[p]->num_groups, rpad, d[p]->in_features, d[p]->out_features);
    J.rpad[p] = rpad;
    per_group = std::max(per_group, (int64_t)rpad * (d[p]->in_features / 8 + 1) + (int64_t)d[p]->out_features * (rpad / 8));
    groups = std::max(groups, d[p]->num_groups);
  }
  const dim3 grid((unsigned)std::min<int64_t>(ceil_div(per_group, 512), 64), (unsigned)groups, (unsigned)n);
  hipLaunchKernelGGL(k_convert_weights, grid, dim3(256), 0, s, J, want_a ? 1 : 0, want_b ? 1 : 0);
  return check_launch();
}

int launch_convert_weights(const tk_lora_desc& d, void* stage, bool want_a, bool want_b, hipStream_t s) {
  const tk_lora_desc* dp = &d;
  return launch_convert_weights_multi(&dp, &stage, 1, want_a, want_b, s);
}

int launch_pass_generic(const PassArgs& a, const SegView& seg, const SegLayout& L, int dtype, int phases,
                        hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  const unsigned grid = (unsigned)L.max_tiles;
  const int32_t* rows = seg.slot_table(a.map_rows);
  const size_t lds_shrink = sizeof(float) * (size_t)(kTileRows + a.rpad) * (kKC + 1);
  const size_t lds_expand = sizeof(float) * (size_t)a.rpad * kTileRows;
  if (dtype == TK_DTYPE_F32) {
    if (phases & 1)
      hipLaunchKernelGGL(k_shrink_generic<float>, dim3(grid), dim3(256), lds_shrink, s, a, seg.tile_group, rows);
    if (a.dst && (phases & 2))
      hipLaunchKernelGGL(k_expand_generic<float>, dim3(grid), dim3(256), lds_expand, s, a, seg.tile_group, rows);
  } else {
    if (phases & 1)
      hipLaunchKernelGGL(k_shrink_generic<bf16_t>, dim3(grid), dim3(256), lds_shrink, s, a, seg.tile_group, rows);
    if (a.dst && (phases & 2))
      hipLaunchKernelGGL(k_expand_generic<bf16_t>, dim3(grid), dim3(256), lds_expand, s, a, seg.tile_group, rows);
  }
  return check_launch();
}

int launch_wgrad_generic(const WgradArgs& a, const SegView& seg, const SegLayout& L, int dtype, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  const dim3 grid((unsigned)L.max_chunks, (unsigned)ceil_div(a.width, 256));
  if (dtype == TK_DTYPE_F32)
    hipLaunchKernelGGL(k_wgrad_generic<float>, grid, dim3(256), 0, s, a, seg.chunks, seg.slot_table(a.map_rows));
  else
    hipLaunchKernelGGL(k_wgrad_generic<bf16_t>, grid, dim3(256), 0, s, a, seg.chunks, seg.slot_table(a.map_rows));
  return check_launch();
}

int launch_wgrad_reduce(const WgradArgs* a0, const WgradArgs* a1, const SegView& seg, const SegLayout& L, int dtype,
                        hipStream_t s) {
  if (L.groups == 0 || (!a0 && !a1)) return TK_OK;
  WgradArgs none{};
  const WgradArgs& x0 = a0 ? *a0 : none;
  const WgradArgs& x1 = a1 ? *a1 : none;
  const int rpad = a0 ? a0->rpad : a1->rpad;
  const int width = std::max(a0 ? a0->width : 0, a1 ? a1->width : 0);
  const dim3 grid((unsigned)L.groups, (unsigned)ceil_div(width, 256), (unsigned)(a1 ? 2 * (rpad / 8) : rpad / 8));
  if (dtype == TK_DTYPE_F32 || x0.grad_f32 || x1.grad_f32)  // (both sets have the gradient type of their descriptor)
    hipLaunchKernelGGL(k_wgrad_reduce<float>, grid, dim3(256), 0, s, x0, x1, rpad, seg.chunk_first, seg.partial_first);
  else
    hipLaunchKernelGGL(k_wgrad_reduce<bf16_t>, grid, dim3(256), 0, s, x0, x1, rpad, seg.chunk_first,
                       seg.partial_first);
  return check_launch();
}

int launch_wgrad_reduce_multi(const WgradArgs* sets, int n, const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.groups == 0 || n == 0) return TK_OK;
  WgradReduceJobs J{};
  J.n = n;
  int width = 0;
  for (int i = 0; i < n; ++i) {
    J.a[i] = sets[i];
    width = std::max(width, sets[i].width);
  }
  const int octets = sets[0].rpad / 8;  // the sets share their padded rank
  const dim3 grid((unsigned)L.groups, (unsigned)ceil_div(width, 256), (unsigned)(octets * n));
  if (sets[0].grad_f32)  // fp32 adapters under bf16 activations (all sets of a call alike)
    hipLaunchKernelGGL(k_wgrad_reduce_multi<float>, grid, dim3(256), 0, s, J, octets, seg.chunk_first,
                       seg.partial_first);
  else
    hipLaunchKernelGGL(k_wgrad_reduce_multi<bf16_t>, grid, dim3(256), 0, s, J, octets, seg.chunk_first,
                       seg.partial_first);
  return check_launch();
}

int launch_transpose_weights(const tk_lora_desc& d, int rank_lo, void* bT, void* aT, hipStream_t s) {
  if (d.num_groups == 0) return TK_OK;
  const int rpad = rank_pad(d.max_rank);
  const int64_t per_group = (int64_t)rpad * (d.out_features + d.in_features);
  const dim3 grid((unsigned)std::min<int64_t>(ceil_div(per_group, 256), 64), (unsigned)d.num_groups);
  if (d.dtype == TK_DTYPE_F32)
    hipLaunchKernelGGL((k_transpose_weights<float, float>), grid, dim3(256), 0, s, d, rpad, rank_lo, (float*)bT,
                       (float*)aT);
  else if (mixed_weights(d))
    hipLaunchKernelGGL((k_transpose_weights<float, bf16_t>), grid, dim3(256), 0, s, d, rpad, rank_lo,
                       (bf16_t*)bT, (bf16_t*)aT);
  else
    hipLaunchKernelGGL((k_transpose_weights<bf16_t, bf16_t>), grid, dim3(256), 0, s, d, rpad, rank_lo, (bf16_t*)bT,
                       (bf16_t*)aT);
  return check_launch();
}

}  // namespace tk
