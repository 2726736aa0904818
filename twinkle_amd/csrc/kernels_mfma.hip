// bf16 kernels for gfx950 built on v_mfma_f32_16x16x32_bf16 (fp32 accumulate).
//
// Both kernels are HBM-streaming: the matrix cores are used because the vector
// ALUs could not keep up with 8 TB/s at these ranks, not because the op is
// compute bound.  Everything is laid out so that each wave-wide load covers
// whole 128-byte lines and every activation byte crosses HBM once per pass.
//
// MFMA operand layout used below (l = lane, 64 lanes):
//   A operand: lane l holds A[i = l % 16][k = 8 * (l / 16) .. + 8]   (8 bf16 = 16 B)
//   B operand: lane l holds B[k = 8 * (l / 16) .. + 8][j = l % 16]
//   D        : lane l holds D[i = 4 * (l / 16) + v][j = l % 16], v = 0..3
// The contraction index k may be permuted freely as long as A and B agree, and
// the output indices i, j may be mapped to any rows / columns: both freedoms
// are used to make the global accesses contiguous.
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
// keep elements [lo, hi) of a quad
__device__ inline uint4 keep_range(uint4 v, int lo, int hi) {
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const bool e0 = (2 * d) >= lo && (2 * d) < hi, e1 = (2 * d + 1) >= lo && (2 * d + 1) < hi;
    w[d] &= (e0 ? 0xffffu : 0u) | (e1 ? 0xffff0000u : 0u);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// ---------------------------------------------------------------------------
// Shrink: h[p][n] = scale_g * sum_k src[row(p)][k] * W1_g[n][k] for one tile of up
// to 32 rows of one group per workgroup.  The NW waves split the source width
// in 64-column steps (interleaved, so the workgroup reads 64*NW contiguous
// columns of each row at a time); every wave keeps its partial h[32][rank] in
// MFMA accumulators, issuing the loads of PF steps before the first MFMA so
// that ~PF*6 KB per wave are in flight.  Partials meet in LDS and are summed
// in wave order (fixed order: bitwise repeatable), scaled, rounded to bf16
// and written twice: position-major (hrow, the expand kernel's A operand) and
// rank-major (hT, read by the weight-gradient kernel).
// ---------------------------------------------------------------------------
template <int NB, int NW, int PF>
__global__ __launch_bounds__(NW * 64) void k_shrink_mfma(PassArgs a, bf16_t* __restrict__ hrow,
                                                         const TileInfo* __restrict__ tiles,
                                                         const int32_t* __restrict__ perm, const SegHeader* hdr) {
  constexpr int RP = 16 * NB;  // padded rank
  constexpr int PR = RP + 1;   // row stride of the partial sums (floats; odd: conflict-free column reads)
  __shared__ float part[NW][kTileRows][PR];

  const int tile_id = blockIdx.x;
  if (tile_id >= hdr->num_tiles) return;
  const TileInfo ti = tiles[tile_id];
  const int g = ti.group;
  const int r = min(a.rank[g], RP);
  if (r <= 0) return;  // adapter not live on this layer
  const int cnt = ti.count;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;

  const int pa = ti.start + min(li, cnt - 1), pb = ti.start + min(16 + li, cnt - 1);
  const int64_t ra = a.map_rows ? perm[pa] : pa, rb = a.map_rows ? perm[pb] : pb;
  const bf16_t* src = (const bf16_t*)a.src;
  const bf16_t* xa = src + ra * a.ld_src + 16 * kb;
  const bf16_t* xb = src + rb * a.ld_src + 16 * kb;
  const bf16_t* W1 = group_weight<bf16_t>(a.w_shrink, a.w_shrink_base, a.shrink_group_stride, g);
  const bf16_t* wp[NB];
  bool wv[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int n = 16 * nb + li;
    wv[nb] = n < r;
    wp[nb] = W1 + (int64_t)(wv[nb] ? n : 0) * a.ld_shrink + 16 * kb;
  }
  f32x4 acc[2][NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    acc[0][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc[1][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int nsteps = a.width_src >> 6;
  for (int s0 = wave; s0 < nsteps; s0 += NW * PF) {
    uint4 xa0[PF], xa1[PF], xb0[PF], xb1[PF], w0[PF][NB], w1[PF][NB];
#pragma unroll
    for (int j = 0; j < PF; ++j) {
      const int s = s0 + j * NW;
      const bool ok = s < nsteps;  // wave-uniform
      const int c = (ok ? s : s0) << 6;
      xa0[j] = ld16(xa + c);
      xa1[j] = ld16(xa + c + 8);
      xb0[j] = ld16(xb + c);
      xb1[j] = ld16(xb + c + 8);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        w0[j][nb] = (wv[nb] && ok) ? ld16(wp[nb] + c) : zero4();
        w1[j][nb] = (wv[nb] && ok) ? ld16(wp[nb] + c + 8) : zero4();
      }
    }
#pragma unroll
    for (int j = 0; j < PF; ++j)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        acc[0][nb] = mfma16(xa0[j], w0[j][nb], acc[0][nb]);
        acc[1][nb] = mfma16(xb0[j], w0[j][nb], acc[1][nb]);
        acc[0][nb] = mfma16(xa1[j], w1[j][nb], acc[0][nb]);
        acc[1][nb] = mfma16(xb1[j], w1[j][nb], acc[1][nb]);
      }
  }
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int v = 0; v < 4; ++v) part[wave][16 * tt + 4 * kb + v][16 * nb + li] = acc[tt][nb][v];
  __syncthreads();

  const float sc = a.scale[g];
  bf16_t* hT = (bf16_t*)a.hT;
  // position-major copy: consecutive threads -> consecutive rank indices of one row
  for (int idx = tid; idx < kTileRows * RP; idx += NW * 64) {
    const int row = idx / RP, n = idx % RP;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += part[w][row][n];
    if (row < cnt) hrow[(int64_t)(ti.start + row) * RP + n] = (bf16_t)(pack_bf16(sum * sc, 0.f) & 0xffffu);
  }
  // rank-major copy: consecutive threads -> consecutive rows of one rank index
  for (int idx = tid; idx < kTileRows * RP; idx += NW * 64) {
    const int n = idx >> 5, row = idx & 31;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += part[w][row][n];
    if (row < cnt) hT[(int64_t)n * a.ldh + ti.start + row] = (bf16_t)(pack_bf16(sum * sc, 0.f) & 0xffffu);
  }
}

// ---------------------------------------------------------------------------
// Expand: dst[row(p)][c] += sum_n h[p][n] * W2_g[c][n], read-modify-write in
// place.  Work is flat: one wave owns CPW adjacent 128-column groups of one
// 32-row tile and nothing is shared between waves, so the grid is thousands
// of independent streams.  Column c0 + 8 j + q of a group is output column j
// of MFMA q, which makes each lane's 8 results of one row 16 contiguous
// bytes and each wave-wide access 4 rows x 256 B.
// ---------------------------------------------------------------------------
template <int NB, int CPW>
__global__ __launch_bounds__(256) void k_expand_mfma(PassArgs a, const bf16_t* __restrict__ hrow,
                                                     const TileInfo* __restrict__ tiles,
                                                     const int32_t* __restrict__ perm, const SegHeader* hdr) {
  constexpr int RP = 16 * NB;
  constexpr int NKS = (RP + 31) / 32;  // contraction steps of the MFMAs
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const int ngroups = a.width_dst >> 7;
  const int items_per_tile = (ngroups + CPW - 1) / CPW;
  const int item = blockIdx.x * 4 + wave;
  const int tile_id = item / items_per_tile;
  if (tile_id >= hdr->num_tiles) return;
  const int cg0 = (item - tile_id * items_per_tile) * CPW;
  const TileInfo ti = tiles[tile_id];
  const int g = ti.group;
  const int r = min(a.rank[g], RP);
  if (r <= 0) return;
  const int cnt = ti.count;

  // rows this lane updates: 16 tt + 4 kb + v
  bf16_t* yp[2][4];
  bool yok[2][4];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int row = 16 * tt + 4 * kb + v;
      yok[tt][v] = row < cnt;
      const int p = ti.start + min(row, cnt - 1);
      const int64_t rr = a.map_rows ? perm[p] : p;
      yp[tt][v] = (bf16_t*)a.dst + rr * a.ld_dst + 8 * li;
    }
  uint4 hop[2][NKS];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const int n0 = 32 * ks + 8 * kb;
      const int p = ti.start + min(16 * tt + li, cnt - 1);
      hop[tt][ks] = n0 < RP ? ld16(hrow + (int64_t)p * RP + n0) : zero4();
    }
  const bf16_t* W2 = group_weight<bf16_t>(a.w_expand, a.w_expand_base, a.expand_group_stride, g);

  uint4 y[CPW][2][4];
  uint4 bq[CPW][8][NKS];
#pragma unroll
  for (int u = 0; u < CPW; ++u) {
    const bool gok = cg0 + u < ngroups;  // wave-uniform
    const int c0 = (gok ? cg0 + u : cg0) << 7;
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int v = 0; v < 4; ++v) y[u][tt][v] = (yok[tt][v] && gok) ? ld16(yp[tt][v] + c0) : zero4();
#pragma unroll
    for (int q = 0; q < 8; ++q)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int n0 = 32 * ks + 8 * kb;
        bq[u][q][ks] =
            n0 < r ? keep_first(ld16(W2 + (int64_t)(c0 + 8 * li + q) * a.ld_expand + n0), r - n0) : zero4();
      }
  }
#pragma unroll
  for (int u = 0; u < CPW; ++u) {
    if (cg0 + u >= ngroups) break;
    const int c0 = (cg0 + u) << 7;
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      f32x4 d[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        d[q] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) d[q] = mfma16(hop[tt][ks], bq[u][q][ks], d[q]);
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        if (!yok[tt][v]) continue;
        const uint4 yy = y[u][tt][v];
        uint4 o;
        o.x = pack_bf16(bf16_lo(yy.x) + d[0][v], bf16_hi(yy.x) + d[1][v]);
        o.y = pack_bf16(bf16_lo(yy.y) + d[2][v], bf16_hi(yy.y) + d[3][v]);
        o.z = pack_bf16(bf16_lo(yy.z) + d[4][v], bf16_hi(yy.z) + d[5][v]);
        o.w = pack_bf16(bf16_lo(yy.w) + d[6][v], bf16_hi(yy.w) + d[7][v]);
        st16(yp[tt][v] + c0, o);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Row contraction (weight gradients): out[n][c] = sum_p hT[n][p] * src[row(p)][c]
// over the rows of one chunk of one group.  One wave owns 128 columns; it
// walks the chunk in 32-row windows aligned to absolute multiples of 32 (so
// the hT loads are 16-byte aligned).  Each lane loads 8 rows x 8 columns
// (eight fully coalesced wave loads of 4 x 256 B), transposes its 8x8 block in
// registers with v_perm_b32 so that rows become the MFMA contraction index,
// and accumulates 128 columns x rank in MFMA registers for the whole chunk.
// ---------------------------------------------------------------------------
template <int NB>
__global__ __launch_bounds__(256) void k_wgrad_mfma(WgradArgs a, const ChunkInfo* __restrict__ chunks,
                                                    const int32_t* __restrict__ perm, const SegHeader* hdr) {
  const int chunk_id = blockIdx.x;
  if (chunk_id >= hdr->num_chunks) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const int c0 = (blockIdx.y * 4 + wave) * 128;
  if (c0 >= a.width) return;
  const ChunkInfo ci = chunks[chunk_id];
  const int g = ci.group;
  const int r = min(a.rank[g], 16 * NB);
  if (r <= 0) return;

  const bf16_t* src = (const bf16_t*)a.src + c0 + 8 * li;
  const bf16_t* hT = (const bf16_t*)a.hT + 8 * kb;
  f32x4 acc[8][NB];
#pragma unroll
  for (int q = 0; q < 8; ++q)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[q][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int w0 = ci.start & ~31; w0 < ci.end; w0 += 32) {
    const int p0 = w0 + 8 * kb;  // first of this lane's 8 rows
    const bool interior = w0 >= ci.start && w0 + 32 <= ci.end;
    int rows[8];
    if (a.map_rows) {
      const int4 ra = *reinterpret_cast<const int4*>(perm + p0);
      const int4 rb = *reinterpret_cast<const int4*>(perm + p0 + 4);
      rows[0] = ra.x; rows[1] = ra.y; rows[2] = ra.z; rows[3] = ra.w;
      rows[4] = rb.x; rows[5] = rb.y; rows[6] = rb.z; rows[7] = rb.w;
    } else {
#pragma unroll
      for (int q = 0; q < 8; ++q) rows[q] = p0 + q;
    }
    uint4 x[8];
    uint4 h[NB];
    if (interior) {
#pragma unroll
      for (int q = 0; q < 8; ++q) x[q] = ld16(src + (int64_t)rows[q] * a.ld_src);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) h[nb] = ld16(hT + (int64_t)(16 * nb + li) * a.ldh + w0);
    } else {
      // first / last window of the chunk: rows outside [start, end) belong to other groups
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const bool ok = p0 + q >= ci.start && p0 + q < ci.end;
        x[q] = ok ? ld16(src + (int64_t)rows[q] * a.ld_src) : zero4();
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        h[nb] = keep_range(ld16(hT + (int64_t)(16 * nb + li) * a.ldh + w0), ci.start - p0, ci.end - p0);
    }
    // 8x8 transpose inside the lane: t[q] holds column q of the 8 rows
    uint4 t[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int d = q >> 1;
      const uint32_t sel = (q & 1) ? 0x07060302u : 0x05040100u;
      uint32_t e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t wsrc[4] = {x[i].x, x[i].y, x[i].z, x[i].w};
        e[i] = wsrc[d];
      }
      t[q].x = __builtin_amdgcn_perm(e[1], e[0], sel);
      t[q].y = __builtin_amdgcn_perm(e[3], e[2], sel);
      t[q].z = __builtin_amdgcn_perm(e[5], e[4], sel);
      t[q].w = __builtin_amdgcn_perm(e[7], e[6], sel);
    }
#pragma unroll
    for (int q = 0; q < 8; ++q)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[q][nb] = mfma16(t[q], h[nb], acc[q][nb]);
  }

  // lane holds out[n = 16 nb + li][c0 + 32 kb + 8 v + q], q = 0..7, v = 0..3: 32 consecutive columns per n
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int n = 16 * nb + li;
    if (n >= r) continue;
    const int cb = c0 + 32 * kb;
    if (ci.partial >= 0) {
      float* o = a.partial + ((int64_t)ci.partial * a.rpad + n) * a.width + cb;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        *reinterpret_cast<float4*>(o + 8 * v) = make_float4(acc[0][nb][v], acc[1][nb][v], acc[2][nb][v], acc[3][nb][v]);
        *reinterpret_cast<float4*>(o + 8 * v + 4) =
            make_float4(acc[4][nb][v], acc[5][nb][v], acc[6][nb][v], acc[7][nb][v]);
      }
    } else {
      bf16_t* gp = (bf16_t*)a.grad[g];
#pragma unroll
      for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const int c = cb + 8 * v + q;
          bf16_t* o = a.transposed ? gp + (int64_t)c * a.ld_grad + n : gp + (int64_t)n * a.ld_grad + c;
          float val = acc[q][nb][v];
          if (a.accumulate) val += to_f32(*o);
          *o = (bf16_t)(pack_bf16(val, 0.f) & 0xffffu);
        }
    }
  }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int NB, int NW, int PF, int CPW>
void launch_pass(const PassArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s) {
  bf16_t* hrow = (bf16_t*)a.hT + (int64_t)a.rpad * a.ldh;  // second half of the h buffer
  hipLaunchKernelGGL((k_shrink_mfma<NB, NW, PF>), dim3((unsigned)L.max_tiles), dim3(NW * 64), 0, s, a, hrow,
                     seg.tiles, seg.perm, seg.header);
  if (!a.dst) return;
  const int64_t ngroups = a.width_dst >> 7;
  const int64_t items = L.max_tiles * ceil_div(ngroups, CPW);
  hipLaunchKernelGGL((k_expand_mfma<NB, CPW>), dim3((unsigned)ceil_div(items, 4)), dim3(256), 0, s, a, hrow,
                     seg.tiles, seg.perm, seg.header);
}

template <int NB>
void launch_wgrad(const WgradArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s) {
  const dim3 grid((unsigned)L.max_chunks, (unsigned)ceil_div(a.width, 512));
  hipLaunchKernelGGL((k_wgrad_mfma<NB>), grid, dim3(256), 0, s, a, seg.chunks, seg.perm, seg.header);
}

}  // namespace

bool pass_mfma_supported(const PassArgs& a) {
  if (a.rpad > 64) return false;
  if (a.width_src % 64 != 0 || a.ld_src % 8 != 0 || !aligned16(a.src)) return false;
  if (a.dst && (a.width_dst % 128 != 0 || a.ld_dst % 8 != 0 || !aligned16(a.dst))) return false;
  if (a.ld_shrink % 8 != 0 || a.ld_expand % 8 != 0 || a.ldh % 8 != 0) return false;
  if (a.w_shrink_base && !aligned16(a.w_shrink_base)) return false;
  if (a.w_expand_base && !aligned16(a.w_expand_base)) return false;
  return true;
}

int launch_pass_mfma(const PassArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  if (a.rpad <= 16) launch_pass<1, 4, 4, 2>(a, seg, L, s);
  else if (a.rpad <= 32) launch_pass<2, 4, 4, 2>(a, seg, L, s);
  else launch_pass<4, 4, 2, 1>(a, seg, L, s);
  return check_launch();
}

bool wgrad_mfma_supported(const WgradArgs& a) {
  if (a.rpad > 64) return false;
  if (a.width % 128 != 0 || a.ld_src % 8 != 0 || a.ldh % 8 != 0 || !aligned16(a.src) || !aligned16(a.hT)) return false;
  return true;
}

int launch_wgrad_mfma(const WgradArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  if (a.rpad <= 16) launch_wgrad<1>(a, seg, L, s);
  else if (a.rpad <= 32) launch_wgrad<2>(a, seg, L, s);
  else launch_wgrad<4>(a, seg, L, s);
  return check_launch();
}

}  // namespace tk
