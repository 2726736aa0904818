// bf16 kernels for gfx950 built on v_mfma_f32_16x16x32_bf16 (fp32 accumulate).
//
// All of these kernels stream activations from HBM: the matrix cores are used
// because the vector ALUs could not keep up with 8 TB/s at these ranks, not
// because anything is compute bound.  Everything is laid out so that each
// wave-wide load covers whole 128-byte lines and every activation byte crosses
// HBM once per pass.
//
//   k_shrink_pair / k_shrink_finish      h = scale * x A^T (split over column slices when x is wide)
//   k_expand_mfma / k_expand_multi       y += h B^T in place (rank <= 16 / above)
//   k_dy_fused<NB>                       backward, rank <= 32: dB and the slices of dh from one pass over dy
//   k_wgrad_pipe / k_wgrad_coop          dA, dB: contraction over the rows of a chunk (rank <= 16 / above)
//   k_transpose_job                      B^T, A^T copies for the backward shrink / expand
//   *_multi                              the same bodies for several projections in one launch
//
// MFMA operand layout used below (l = lane, 64 lanes):
//   A operand: lane l holds A[i = l % 16][k = 8 * (l / 16) .. + 8]   (8 bf16 = 16 B)
//   B operand: lane l holds B[k = 8 * (l / 16) .. + 8][j = l % 16]
//   D        : lane l holds D[i = 4 * (l / 16) + v][j = l % 16], v = 0..3
// The contraction index k may be permuted freely as long as A and B agree, and
// the output indices i, j may be mapped to any rows / columns: both freedoms
// are used to make the global accesses contiguous.
#include <algorithm>

#include "tk_mfma.h"

// depths of the software pipelines of k_dy_fused<1>, k_dy_fused<2> (one tile: with two blocks of accumulators a second
// tile in registers leaves one wave per SIMD), k_wgrad_pipe<1, S> and k_wgrad_coop<NB, S> (tiles in registers per wave)
#ifndef TK_DY_STAGES
#define TK_DY_STAGES 2
#endif
#ifndef TK_DY_STAGES2
#define TK_DY_STAGES2 1
#endif
#ifndef TK_COOP_STAGES
#define TK_COOP_STAGES 3
#endif
#ifndef TK_WGRAD_STAGES
#define TK_WGRAD_STAGES 3
#endif

// pairs of waves per block of k_wgrad_coop (see wgrad_coop_body)
#ifndef TK_COOP_PAIRS
#define TK_COOP_PAIRS 2
#endif

// h operands of k_expand_multi through LDS (once per block) or straight from memory (once per wave)
#ifndef TK_EXPAND_LDS_H
#define TK_EXPAND_LDS_H 1
#endif

// block renumbering of the rank > 16 expand (contiguous runs of tiles per XCD)
#ifndef TK_XCD_MAP
#define TK_XCD_MAP(b, n) xcd_contiguous(b, n)
#endif

namespace tk {

namespace {

// Scales, rounds and writes one tile of h from `planes` partial planes in LDS ([plane][32][RP + 1]):
// slot-major (hrow) and rank-major (hT); padding slots (row >= cnt) get exact zeros.
template <int RP, int THREADS>
__device__ inline void shrink_epilogue(const float* part, int planes, const PassArgs& a, bf16_t* __restrict__ hrow,
                                       int slot0, int cnt, float sc) {
  constexpr int PR = RP + 1;
  const int tid = threadIdx.x;
  bf16_t* hT = (bf16_t*)a.hT;
  // slot-major copy: consecutive threads -> consecutive rank indices of one slot
  for (int idx = tid; idx < kTileRows * RP; idx += THREADS) {
    const int row = idx / RP, n = idx % RP;
    float sum = 0.f;
    for (int w = 0; w < planes; ++w) sum += part[(w * kTileRows + row) * PR + n];
    hrow[(int64_t)(slot0 + row) * RP + n] = row < cnt ? (bf16_t)(pack_bf16(sum * sc, 0.f) & 0xffffu) : (bf16_t)0;
  }
  // rank-major copy: consecutive threads -> consecutive slots of one rank index
  for (int idx = tid; idx < kTileRows * RP; idx += THREADS) {
    const int n = idx >> 5, row = idx & 31;
    float sum = 0.f;
    for (int w = 0; w < planes; ++w) sum += part[(w * kTileRows + row) * PR + n];
    hT[(int64_t)n * a.ldh + slot0 + row] = row < cnt ? (bf16_t)(pack_bf16(sum * sc, 0.f) & 0xffffu) : (bf16_t)0;
  }
}

// ---------------------------------------------------------------------------
// Shrink: h[slot][n] = scale_g * sum_k src[row(slot)][k] * W1_g[n][k].
//
// Work item = (two consecutive tiles of 32 padded slots, slice of 512*NW source columns), one block of
// NW waves; the slices of a tile pair are consecutive blocks, so neighbouring waves read neighbouring
// 1 KB pieces of the same rows.  The grid is thousands of short independent streams: the hardware
// dispatcher keeps every CU equally loaded, which a tile-per-workgroup split does not (2.03 workgroups
// per CU leaves most CUs waiting for the few that got 3).  A wave takes 64-column steps, interleaved
// with the other waves of its block, keeps its partial h[32][rank] of both tiles in MFMA accumulators
// and issues the loads of two steps before the first MFMA of the batch.  Every weight operand feeds both
// tiles: at rank 64 a step has 8 weight loads for 4 source loads per tile, and with one tile per block the
// load pipeline, not memory, set the pace (rank 64: 129 -> 87 us; rank 16: 2 us).  Consecutive tiles
// almost always belong to the same group; a pair that straddles a group boundary is done one tile at a
// time.  The waves' partials meet in LDS; if the source is wider than one block the block sums go to
// a global buffer and k_shrink_finish adds the slices in slice order (a device-scope fence per block,
// the alternative, costs a cache write-back on this multi-die part).  Summation order is fixed
// throughout: results are bitwise repeatable.  The result is scaled, rounded to bf16 and written
// twice: slot-major (hrow, the expand kernel's A operand) and rank-major (hT, read by the
// weight-gradient kernels); padding slots get exact zeros.
// ---------------------------------------------------------------------------
template <int NB, int NW, int TT>
__device__ inline void shrink_tiles(const PassArgs& a, bf16_t* __restrict__ hrow, const int32_t* __restrict__ slot_rows,
                                    const int (&tiles)[TT], int g, int ks, float (*part)[kTileRows][16 * NB + 1]) {
  constexpr int RP = 16 * NB;
  constexpr int PF = 2;  // steps whose loads are issued together
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const bf16_t* src = (const bf16_t*)a.src;
  const bf16_t *xa[TT], *xb[TT];
  int cnt[TT];
#pragma unroll
  for (int u = 0; u < TT; ++u) {
    const int slot0 = tiles[u] * kTileRows;
    int ra = slot_rows[slot0 + li], rb = slot_rows[slot0 + 16 + li];
    // padding is always at the end of a tile: count the valid slots
    cnt[u] = __popcll(__ballot(ra >= 0) & 0xffffull) + __popcll(__ballot(rb >= 0) & 0xffffull);
    ra = min(max(ra, 0), a.src_rows - 1);
    rb = min(max(rb, 0), a.src_rows - 1);
    xa[u] = src + (int64_t)ra * a.ld_src + 16 * kb;
    xb[u] = src + (int64_t)rb * a.ld_src + 16 * kb;
  }
  const int r = class_rank(a.rank[g], a.rank_lo, RP);
  if (a.class_mode && r <= 0) return;  // a group of another rank class (uniform over the block): nothing is requested
  const bf16_t* W1 = group_weight<bf16_t>(a.w_shrink, a.w_shrink_base, a.shrink_group_stride, g);
  const bf16_t* wp[NB];
  bool wv[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int n = 16 * nb + li;
    wv[nb] = n < r;
    wp[nb] = W1 + (int64_t)(wv[nb] ? n : 0) * a.ld_shrink + 16 * kb;
  }
  f32x4 acc[TT][2][NB];
#pragma unroll
  for (int u = 0; u < TT; ++u)
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[u][tt][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int nsteps = a.width_src >> 6;
  const int s_first = ks * (kShrinkSteps * NW) + wave;
#pragma unroll
  for (int b = 0; b < kShrinkSteps / PF; ++b) {
    uint4 x0[PF][TT][2], x1[PF][TT][2], w0[PF][NB], w1[PF][NB];
#pragma unroll
    for (int j = 0; j < PF; ++j) {
      const int s = s_first + (b * PF + j) * NW;
      const bool ok = s < nsteps;  // wave-uniform
      const int c = (ok ? s : 0) << 6;
#pragma unroll
      for (int u = 0; u < TT; ++u) {
        x0[j][u][0] = ld16(xa[u] + c);
        x1[j][u][0] = ld16(xa[u] + c + 8);
        x0[j][u][1] = ld16(xb[u] + c);
        x1[j][u][1] = ld16(xb[u] + c + 8);
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        w0[j][nb] = (wv[nb] && ok) ? ld16(wp[nb] + c) : zero4();
        w1[j][nb] = (wv[nb] && ok) ? ld16(wp[nb] + c + 8) : zero4();
      }
    }
#pragma unroll
    for (int j = 0; j < PF; ++j)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int u = 0; u < TT; ++u)
#pragma unroll
          for (int tt = 0; tt < 2; ++tt) {
            acc[u][tt][nb] = mfma16(x0[j][u][tt], w0[j][nb], acc[u][tt][nb]);
            acc[u][tt][nb] = mfma16(x1[j][u][tt], w1[j][nb], acc[u][tt][nb]);
          }
  }
  if (r <= 0) return;  // adapter not live on this layer (uniform over the block)
  const float sc = a.scale[g];
#pragma unroll
  for (int u = 0; u < TT; ++u) {
    __syncthreads();  // the previous tile's sums have been read
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int v = 0; v < 4; ++v) part[wave][16 * tt + 4 * kb + v][16 * nb + li] = acc[u][tt][nb][v];
    __syncthreads();
    if (a.kslices > 1) {
      // the source is wider than one block: leave this block's sums for k_shrink_finish
      float* mine = a.hpart + ((int64_t)tiles[u] * a.kslices + ks) * (kTileRows * RP);
      for (int idx = tid; idx < kTileRows * RP; idx += NW * 64) {
        const int row = idx / RP, n = idx % RP;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += part[w][row][n];
        mine[idx] = sum;
      }
    } else {
      shrink_epilogue<RP, NW * 64>(&part[0][0][0], NW, a, hrow, tiles[u] * kTileRows, cnt[u], sc);
    }
  }
}

template <int NB, int NW>
__device__ __forceinline__ void shrink_pair_body(const PassArgs& a, bf16_t* __restrict__ hrow,
                                                 const int32_t* __restrict__ tile_group,
                                                 const int32_t* __restrict__ slot_rows, int max_tiles, int item) {
  __shared__ float part[NW][kTileRows][16 * NB + 1];
  const int nth = item / a.kslices, ks = item - nth * a.kslices;
  const int pair = work_item(a.wl_pairs, nth);
  if (pair < 0) return;  // past the end of this rank class's list (uniform over the block)
  const int t0 = 2 * pair, t1 = t0 + 1;
  if (t0 >= max_tiles) return;
  const int g0 = checked_group(tile_group[t0], a.tb);
  const int g1 = t1 < max_tiles ? checked_group(tile_group[t1], a.tb) : -1;
  if (g0 >= 0 && g1 == g0) {
    const int tiles[2] = {t0, t1};
    shrink_tiles<NB, NW, 2>(a, hrow, slot_rows, tiles, g0, ks, part);
    return;
  }
  if (g0 >= 0) {
    const int tiles[1] = {t0};
    shrink_tiles<NB, NW, 1>(a, hrow, slot_rows, tiles, g0, ks, part);
  }
  if (g1 >= 0) {
    const int tiles[1] = {t1};
    shrink_tiles<NB, NW, 1>(a, hrow, slot_rows, tiles, g1, ks, part);
  }
}

template <int NB, int NW>
__global__ __launch_bounds__(NW * 64) void k_shrink_pair(PassArgs a, bf16_t* __restrict__ hrow,
                                                         const int32_t* __restrict__ tile_group,
                                                         const int32_t* __restrict__ slot_rows, int max_tiles) {
  shrink_pair_body<NB, NW>(a, hrow, tile_group, slot_rows, max_tiles, blockIdx.x);
}

// Work item `item` of projection p out of nproj that read the same rows: blocks go to the eight XCDs (each with an
// L2 of its own) round-robin by block number, so the items are numbered in runs of eight per projection: blocks
// 8 (g nproj + p) + j, j < 8, are items 8 g + j of projection p.  The nproj blocks that read the same piece of the
// source then lie eight apart, run on the same XCD at about the same time, and the piece comes from memory once and
// from that L2 afterwards.
__device__ inline void shared_source_item(int block, int nproj, int& p, int& item) {
  const int run = block >> 3;
  p = run % nproj;
  item = ((run / nproj) << 3) + (block & 7);
}

// The shrink of up to kMaxShared projections of one padded rank that read the same source, in one launch: the
// bodies of k_shrink_pair, every piece of the source crossing memory once (see shared_source_item).
template <int NB, int NW>
__global__ __launch_bounds__(NW * 64) void k_shrink_pair_multi(PassJobs jobs, int nproj, int items,
                                                               const int32_t* __restrict__ tile_group,
                                                               const int32_t* __restrict__ slot_rows, int max_tiles) {
  int p, item;
  shared_source_item(blockIdx.x, nproj, p, item);
  if (item >= items) return;
  const PassArgs& a = jobs.p[p];
  shrink_pair_body<NB, NW>(a, (bf16_t*)a.hT + (int64_t)a.rpad * a.ldh, tile_group, slot_rows, max_tiles, item);
}

// ---------------------------------------------------------------------------
// Shrink with the weights shared through LDS, for groups of many tiles.  In k_shrink_pair every wave fetches the
// weight columns of its own steps, 16 * NB rank indices for 64 rows: at rank 64 as many bytes of weights (from L2)
// as of activations (from memory), and the two share the path between L2 and the CUs, which is what sets the pace
// (measured at rank 64: 536 MB of L2 reads for 268 MB of activations, 7.6 TB/s together).  Here a block of four
// waves owns (eight consecutive tiles, slice of 64 * STEPS columns): wave w takes tiles 2 w and 2 w + 1 of the
// eight through all steps, and the weight block of a step (16 * NB x 64) is fetched once per block, 16 B per
// thread, into a double-buffered LDS tile from which every wave reads its MFMA operands: a quarter of the weight
// traffic.  One LDS-only barrier per step: a buffer is overwritten one step after the barrier behind its last
// reader.  The eight tiles are taken in runs of equal group (almost always one run); waves whose tiles lie
// outside the run still help to stage the weights.  The slice length (a.quad_steps) is chosen per launch.  Activations: three steps in registers per wave, loads two
// steps ahead.  Every block leaves its sums as one slice of the split-shrink buffer (k_shrink_finish follows);
// each entry is the sum of one wave's MFMA chain, so results do not depend on timing.
// ---------------------------------------------------------------------------
template <int NB>
__device__ __forceinline__ void shrink_quad_body(const PassArgs& a, const int32_t* __restrict__ tile_group,
                                                 const int32_t* __restrict__ slot_rows, int max_tiles, int item) {
  constexpr int RP = 16 * NB;
  constexpr int WS = 72;                    // row stride of a staged weight block in bf16 (144 B: conflict-free)
  constexpr int NLD = (RP * 8 + 255) / 256;  // 16-byte pieces of a weight block per thread
  constexpr int S = NB == 4 ? 2 : 3;  // steps of activations in registers (rank 64: the accumulators take the room)
  __shared__ __attribute__((aligned(16))) bf16_t wbuf[2][RP * WS];
  __shared__ int32_t gts[8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const int nth = item / a.kslices, ks = item - nth * a.kslices;
  const int set = work_item(a.wl_octs, nth);
  if (set < 0) return;  // past the end of this rank class's list (uniform over the block)
  const int t_first = set * 8;
  if (tid < 8) gts[tid] = t_first + tid < max_tiles ? checked_group(tile_group[t_first + tid], a.tb) : -1;
  const int nsteps = a.width_src >> 6;
  const int s0 = ks * a.quad_steps;
  const int ns = min(a.quad_steps, nsteps - s0);  // >= 1 for every slice
  // this wave's two tiles
  const bf16_t* src = (const bf16_t*)a.src;
  const bf16_t *xa[2], *xb[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int t = min(t_first + 2 * wave + u, max_tiles - 1);
    int ra = slot_rows[t * kTileRows + li], rb = slot_rows[t * kTileRows + 16 + li];
    ra = min(max(ra, 0), a.src_rows - 1);
    rb = min(max(rb, 0), a.src_rows - 1);
    xa[u] = src + (int64_t)ra * a.ld_src + 16 * kb + (int64_t)s0 * 64;
    xb[u] = src + (int64_t)rb * a.ld_src + 16 * kb + (int64_t)s0 * 64;
  }
  __syncthreads();
  for (int j = 0; j < 8;) {
    const int g = gts[j];
    int e = j + 1;
    while (e < 8 && gts[e] == g) ++e;
    const int lo = j, hi = e;  // the run: tiles t_first + lo .. t_first + hi - 1, all of group g
    j = e;
    if (g < 0) continue;
    const int r = class_rank(a.rank[g], a.rank_lo, RP);
    if (r <= 0) continue;  // adapter not live on this layer, or a group of another rank class
    bool mine[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) mine[u] = 2 * wave + u >= lo && 2 * wave + u < hi;
    const bool active = mine[0] || mine[1];  // wave-uniform
    const bf16_t* W1 = group_weight<bf16_t>(a.w_shrink, a.w_shrink_base, a.shrink_group_stride, g) + (int64_t)s0 * 64;
    // staging: piece p = tid + 256 i is columns 8 (p % 8) .. + 8 of rank index p / 8
    auto stage_load = [&](int s, uint4 (&wr)[NLD]) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int p = tid + 256 * i, n = p >> 3;
        wr[i] = (n < r && s < ns) ? ld16(W1 + (int64_t)n * a.ld_shrink + (s << 6) + 8 * (p & 7)) : zero4();
      }
    };
    auto stage_store = [&](int buf, const uint4 (&wr)[NLD]) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int p = tid + 256 * i, n = p >> 3;
        if (n < RP) st16(&wbuf[buf][n * WS + 8 * (p & 7)], wr[i]);
      }
    };
    struct Step {
      uint4 x0[2][2], x1[2][2];
    };
    auto issue = [&](int s, Step& X) {
      const int c = min(s, ns - 1) << 6;  // requests past the slice repeat its last step and are not used
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        X.x0[u][0] = ld16(xa[u] + c);
        X.x1[u][0] = ld16(xa[u] + c + 8);
        X.x0[u][1] = ld16(xb[u] + c);
        X.x1[u][1] = ld16(xb[u] + c + 8);
      }
    };
    f32x4 acc[2][2][NB];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[u][tt][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
    uint4 wr[NLD];
    auto step = [&](int s, const Step& X, Step& Xnext) {
      lds_barrier();  // block s is complete; the other buffer has been read by everyone
      stage_load(s + 1, wr);
      if (active) issue(s + S - 1, Xnext);
      if (active) {
        const bf16_t* wb = wbuf[s & 1] + li * WS + 16 * kb;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const uint4 w0 = ld16(wb + 16 * nb * WS), w1 = ld16(wb + 16 * nb * WS + 8);
#pragma unroll
          for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
              acc[u][tt][nb] = mfma16(X.x0[u][tt], w0, acc[u][tt][nb]);
              acc[u][tt][nb] = mfma16(X.x1[u][tt], w1, acc[u][tt][nb]);
            }
        }
      }
      stage_store((s + 1) & 1, wr);  // block s + 1 (zeros past the slice), visible behind the next barrier
    };
    Step T[S];
    stage_load(0, wr);
    if (active) {
#pragma unroll
      for (int i = 0; i < S - 1; ++i) issue(i, T[i]);
    }
    stage_store(0, wr);
    int s = 0;
    for (; s + S <= ns; s += S) {
#pragma unroll
      for (int i = 0; i < S; ++i) step(s + i, T[i], T[(i + S - 1) % S]);
    }
#pragma unroll
    for (int i = 0; i < S - 1; ++i)
      if (s + i < ns) step(s + i, T[i], T[(i + S - 1) % S]);  // block-uniform
    lds_barrier();  // the next run's first block goes into buffer 0
    if (!active) continue;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      if (!mine[u]) continue;
      float* out = a.hpart + ((int64_t)(t_first + 2 * wave + u) * a.kslices + ks) * (kTileRows * RP) + 4 * kb * RP + li;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int v = 0; v < 4; ++v) out[(16 * tt + v) * RP + 16 * nb] = acc[u][tt][nb][v];
    }
  }
}

template <int NB>
__global__ __launch_bounds__(256, 2) void k_shrink_quad(PassArgs a, const int32_t* __restrict__ tile_group,
                                                     const int32_t* __restrict__ slot_rows, int max_tiles) {
  shrink_quad_body<NB>(a, tile_group, slot_rows, max_tiles, blockIdx.x);
}

// The same for up to kMaxShared projections that read the same source (see shared_source_item).
template <int NB>
__global__ __launch_bounds__(256, 2) void k_shrink_quad_multi(PassJobs jobs, int nproj, int items,
                                                           const int32_t* __restrict__ tile_group,
                                                           const int32_t* __restrict__ slot_rows, int max_tiles) {
  int p, item;
  shared_source_item(blockIdx.x, nproj, p, item);
  if (item >= items) return;
  shrink_quad_body<NB>(jobs.p[p], tile_group, slot_rows, max_tiles, item);
}

// Adds the slices of a split shrink in slice order and writes h (one block per tile).
template <int NB>
__device__ __forceinline__ void shrink_finish_body(const PassArgs& a, bf16_t* __restrict__ hrow,
                                                   const int32_t* __restrict__ tile_group,
                                                   const int32_t* __restrict__ slot_rows, int nth) {
  constexpr int RP = 16 * NB, PR = RP + 1;
  __shared__ float part[kTileRows][PR];
  const int tid = threadIdx.x;
  const int tile_id = checked_tile(work_item(a.wl_tiles, nth), a.tb);
  if (tile_id < 0) return;  // past the end of this rank class's list
  const int slot0 = tile_id * kTileRows;
  // independent loads first: group id, this tile's row indices, the slices themselves
  const int g = checked_group(tile_group[tile_id], a.tb);
  // (with several rank classes most tiles belong to another launch: look before reading their slices)
  if (a.class_mode && (g < 0 || class_rank(a.rank[g], a.rank_lo, RP) <= 0)) return;
  const int my_row = slot_rows[slot0 + (tid & 31)];
  const float* tile_part = a.hpart + (int64_t)tile_id * a.kslices * (kTileRows * RP);
  constexpr int NI = (kTileRows * RP + 255) / 256;
  float sums[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) sums[i] = 0.f;
  // eight slices are requested together (their latencies overlap) and added in slice order
  for (int k0 = 0; k0 < a.kslices; k0 += 8) {
    float v[NI][8];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int idx = tid + 256 * i;
#pragma unroll
      for (int k = 0; k < 8; ++k)
        v[i][k] = (idx < kTileRows * RP && k0 + k < a.kslices) ? tile_part[(int64_t)(k0 + k) * (kTileRows * RP) + idx] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int k = 0; k < 8; ++k) sums[i] += v[i][k];
  }
  const int gg = max(g, 0);
  const int rk = class_rank(a.rank[gg], a.rank_lo, RP);
  const float sc = a.scale[gg];
  if (g < 0 || rk <= 0) return;
  const int cnt = __popcll(__ballot(my_row >= 0) & 0xffffffffull);  // padding is at the end of a tile
#pragma unroll
  for (int i = 0; i < (kTileRows * RP + 255) / 256; ++i) {
    const int idx = tid + 256 * i;
    if (idx < kTileRows * RP) part[idx / RP][idx % RP] = sums[i];
  }
  __syncthreads();
  shrink_epilogue<RP, 256>(&part[0][0], 1, a, hrow, slot0, cnt, sc);
}

template <int NB>
__global__ __launch_bounds__(256) void k_shrink_finish(PassArgs a, bf16_t* __restrict__ hrow,
                                                       const int32_t* __restrict__ tile_group,
                                                       const int32_t* __restrict__ slot_rows) {
  shrink_finish_body<NB>(a, hrow, tile_group, slot_rows, blockIdx.x);
}

// The same for up to kMaxShared projections of padded rank 16 in one launch: blockIdx.y selects the projection.
__global__ __launch_bounds__(256) void k_shrink_finish_multi(PassJobs jobs, const int32_t* __restrict__ tile_group,
                                                             const int32_t* __restrict__ slot_rows) {
  const PassArgs& a = jobs.p[blockIdx.y];
  shrink_finish_body<1>(a, (bf16_t*)a.hT + (int64_t)a.rpad * a.ldh, tile_group, slot_rows, blockIdx.x);
}

// ---------------------------------------------------------------------------
// Expand: dst[row(slot)][c] += sum_n h[slot][n] * W2_g[c][n], read-modify-write
// in place.  Work is flat: one wave owns one 128-column group of one tile and
// nothing is shared between waves, so the grid is thousands of independent
// streams.  Column c0 + 8 j + q of a group is output column j of MFMA q, which
// makes each lane's 8 results of one row 16 contiguous bytes and each wave-wide
// access 4 rows x 256 B.  Row indices, h and the group id are addressed from the
// work-item number alone, so the destination loads are one dependent step away
// from the start of the wave.  (Used for padded rank 16; above that
// k_expand_multi shares the weight block between tiles.)
// ---------------------------------------------------------------------------
template <int NB>
__device__ __forceinline__ void expand_flat_body(const PassArgs& a, const bf16_t* __restrict__ hrow,
                                                 const int32_t* __restrict__ tile_group,
                                                 const int32_t* __restrict__ slot_rows,
                                                 const int32_t* __restrict__ tile_walk, int num_items, int block) {
  constexpr int RP = 16 * NB;
  constexpr int NKS = (RP + 31) / 32;  // contraction steps of the MFMAs
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const int ngroups = a.width_dst >> 7;
  const int item = block * 4 + wave;
  if (item >= num_items) return;
  // Items are numbered tile by tile; with a walk order the n-th tile taken is tile_walk[n], the tiles sorted by their
  // first row.  The table itself is group-major and a group's tiles are spread over all rows, so in table order the
  // waves in flight at any moment touch rows all over the destination; in walk order they touch neighbouring rows,
  // and the in-place update runs faster (probe: 43 us against 54 us for 256 MB touched in tiles of 32 random rows
  // taken from windows of 512 rows instead of from all 16384).
  const int nth = item / ngroups;
  // (one of several rank classes: the class's own list of tiles, which is in the same walk order)
  const int tile_id = checked_tile(a.wl_tiles.ids ? work_item(a.wl_tiles, nth) : (tile_walk ? tile_walk[nth] : nth), a.tb);
  if (tile_id < 0) return;
  const int c0 = (item - nth * ngroups) << 7;
  const int slot0 = tile_id * kTileRows;
  // independent first loads: group id, row indices, h operand (nothing branches before the
  // destination loads are in flight)
  const int g_raw = checked_group(tile_group[tile_id], a.tb);
  // rows this lane updates: slots 16 tt + 4 kb + v
  const int4 r0 = *reinterpret_cast<const int4*>(slot_rows + slot0 + 4 * kb);
  const int4 r1 = *reinterpret_cast<const int4*>(slot_rows + slot0 + 16 + 4 * kb);
  uint4 hop[2][NKS];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const int n0 = 32 * ks + 8 * kb;
      hop[tt][ks] = n0 < RP ? ld16(hrow + (int64_t)(slot0 + 16 * tt + li) * RP + n0) : zero4();
    }
  const int g = max(g_raw, 0);
  const int rows[2][4] = {{r0.x, r0.y, r0.z, r0.w}, {r1.x, r1.y, r1.z, r1.w}};
  bool rok[2][4];
  bf16_t* yp[2][4];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      rok[tt][v] = g_raw >= 0 && checked_row(rows[tt][v], a.tb) >= 0;
      yp[tt][v] = (bf16_t*)a.dst + (int64_t)(rok[tt][v] ? rows[tt][v] : 0) * a.ld_dst + 8 * li + c0;
    }
  const int r = g_raw < 0 ? 0 : class_rank(a.rank[g], a.rank_lo, RP);
  if (a.class_mode && r <= 0) return;  // a tile of another rank class: its rows are not even requested
  const bf16_t* W2 = group_weight<bf16_t>(a.w_expand, a.w_expand_base, a.expand_group_stride, g);
  uint4 y[2][4];
  uint4 bq[8][NKS];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int v = 0; v < 4; ++v) y[tt][v] = rok[tt][v] ? ld16_nt(yp[tt][v]) : zero4();
#pragma unroll
  for (int q = 0; q < 8; ++q)
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const int n0 = 32 * ks + 8 * kb;
      const int wrow = a.expand_swizzled ? c0 + 16 * q + li : c0 + 8 * li + q;
      bq[q][ks] = n0 < r ? keep_first(ld16(W2 + (int64_t)wrow * a.ld_expand + n0), r - n0) : zero4();
    }
  if (r <= 0) return;  // unused tile, or adapter not live on this layer (uniform over the wave)
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    f32x4 d[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      d[q] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) d[q] = mfma16(hop[tt][ks], bq[q][ks], d[q]);
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      if (!rok[tt][v]) continue;
      const uint4 yy = y[tt][v];
      uint4 o;
      o.x = pack_bf16(bf16_lo(yy.x) + d[0][v], bf16_hi(yy.x) + d[1][v]);
      o.y = pack_bf16(bf16_lo(yy.y) + d[2][v], bf16_hi(yy.y) + d[3][v]);
      o.z = pack_bf16(bf16_lo(yy.z) + d[4][v], bf16_hi(yy.z) + d[5][v]);
      o.w = pack_bf16(bf16_lo(yy.w) + d[6][v], bf16_hi(yy.w) + d[7][v]);
      st16_nt(yp[tt][v], o);
    }
  }
}

template <int NB>
__global__ __launch_bounds__(256) void k_expand_mfma(PassArgs a, const bf16_t* __restrict__ hrow,
                                                     const int32_t* __restrict__ tile_group,
                                                     const int32_t* __restrict__ slot_rows,
                                                     const int32_t* __restrict__ tile_walk, int num_items) {
  expand_flat_body<NB>(a, hrow, tile_group, slot_rows, tile_walk, num_items, blockIdx.x);
}

// Up to kMaxShared projections of padded rank 16 in one launch: blockIdx.y selects the projection; the grid
// is as wide as the widest projection needs.
__global__ __launch_bounds__(256) void k_expand_mfma_multi(PassJobs jobs, const int32_t* __restrict__ tile_group,
                                                           const int32_t* __restrict__ slot_rows,
                                                           const int32_t* __restrict__ tile_walk, int max_tiles) {
  const PassArgs& a = jobs.p[blockIdx.y];
  expand_flat_body<1>(a, (const bf16_t*)a.hT + (int64_t)a.rpad * a.ldh, tile_group, slot_rows, tile_walk,
                      max_tiles * (a.width_dst >> 7), blockIdx.x);
}

// ---------------------------------------------------------------------------
// Expand for padded ranks above 16.  There a wave's block of W2 (128 columns x rank) is as large as
// its piece of a 32-row tile (16 KB at rank 64), so re-reading it for every tile doubles the traffic
// between L2 and the CUs.  Here a wave keeps the block in registers and walks TPI consecutive tiles:
// work item = (TPI tiles, 128 columns).  Consecutive tiles almost always belong to the same group;
// where the group changes inside an item the wave reloads the block.  The next tile's rows, h operand
// and destination rows are requested before the current tile is consumed.
// ---------------------------------------------------------------------------
// CLS: the launch serves one of several rank classes (work list of sets, ranks outside the class skipped).  A
// compile-time switch because this kernel's schedule is touchy: with the two forms in one body the single-class
// launch measured 10 % slower (config 5's q projection: 116 against 106 us).
template <int NB, int TPI, bool CLS>
__global__ __launch_bounds__(256) void k_expand_multi(PassArgs a, const bf16_t* __restrict__ hrow,
                                                      const int32_t* __restrict__ tile_group,
                                                      const int32_t* __restrict__ slot_rows,
                                                      const int32_t* __restrict__ set_walk,
                                                      const SegHeader* __restrict__ header,
                                                      const uint8_t* __restrict__ round_moved, int sort_blocks,
                                                      int max_tiles) {
  static_assert(TPI == kSetTiles, "the segment table's set order is built for sets of kSetTiles tiles");
  constexpr int RP = 16 * NB;
  constexpr int NKS = (RP + 31) / 32;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const int ngroups = a.width_dst >> 7;
  const int nbt = (ngroups + 3) >> 2;  // blocks per tile set: column block fastest
  // Gathered rows whose groups interleave: the sets of tiles in the order of their first row, so that neighbouring
  // rows are in flight together (measured at config 3: 2.5 % of the step).  Rows in segment order, or a table built
  // from keys that came in order (then that order is the identity): contiguous runs of sets per XCD, whose L2 then
  // fetches the weights of few groups (1.2 % at config 5's q projection; combining the two loses the first gain).
  // Whether the keys came in order is in the builder's flags, one byte per 64 rows, eight per lane here.
  // (the flags and the order entry are requested together: one round trip in front of the tile's first loads)
  int swept_set = 0;
  bool sweep = false;
  if constexpr (CLS) {
    // the class's list of sets, already in the order to take them in
    swept_set = work_item(a.wl_sets, blockIdx.x / nbt);
    if (swept_set < 0) return;
    sweep = true;
  } else if (set_walk != nullptr) {
    swept_set = set_walk[blockIdx.x / nbt];
    uint2 moved = make_uint2(0u, 0u);
    if (lane < sort_blocks) moved = reinterpret_cast<const uint2*>(round_moved)[lane];
    sweep = header->identity_order == 0 && __ballot((moved.x | moved.y) != 0u) != 0ull;
  }
  const int block = sweep ? (int)blockIdx.x : TK_XCD_MAP(blockIdx.x, gridDim.x);
  const int cb = block % nbt, set = block / nbt;
  const int tile0 = (sweep ? swept_set : set) * TPI;
  const int cg = cb * 4 + wave;
  if ((unsigned)tile0 >= (unsigned)max_tiles) return;  // (uniform over the block)
  const int nt = min(TPI, max_tiles - tile0);
  int gt[TPI];
#pragma unroll
  for (int t = 0; t < TPI; ++t) gt[t] = t < nt ? checked_group(tile_group[tile0 + t], a.tb) : -1;
#if TK_EXPAND_LDS_H
  // The block's four waves multiply the same tiles' h operands with their own columns' weights: the operands (one
  // contiguous run of hrow, nt x 32 slots x RP) are fetched once per block into LDS instead of once per wave.  Row
  // stride RP + 8 elements: operand reads without bank conflicts.
  constexpr int HS = RP + 8;
  __shared__ __attribute__((aligned(16))) bf16_t h_s[TPI * kTileRows * HS];
  {
    constexpr int PPR = RP / 8, PIECES = TPI * kTileRows * PPR, PER = (PIECES + 255) / 256;
    const bf16_t* hp = hrow + (int64_t)tile0 * kTileRows * RP;
    uint4 v[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = tid + 256 * i;
      v[i] = e < nt * kTileRows * PPR ? ld16(hp + 8 * e) : zero4();
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = tid + 256 * i;
      if (e < PIECES) st16(&h_s[(e / PPR) * HS + 8 * (e % PPR)], v[i]);
    }
  }
  __syncthreads();
#endif
  if (cg >= ngroups) return;  // a column group past the width
  const int c0 = cg << 7;
  bf16_t* dst = (bf16_t*)a.dst + c0 + 8 * li;

  struct Tile {
    int rows[2][4];
#if !TK_EXPAND_LDS_H
    uint4 hop[2][NKS];
#endif
    uint4 y[2][4];
    int t;
  };
  auto issue = [&](int t, Tile& T) {
    const bool tok = t < nt;  // wave-uniform
    const unsigned row_limit = tok ? (unsigned)a.tb.rows : 0u;  // rows of the table are in [0, rows): see TableBounds
    const int slot0 = (tile0 + (tok ? t : 0)) * kTileRows;
    const int4 r0 = *reinterpret_cast<const int4*>(slot_rows + slot0 + 4 * kb);
    const int4 r1 = *reinterpret_cast<const int4*>(slot_rows + slot0 + 16 + 4 * kb);
    const int rr[2][4] = {{r0.x, r0.y, r0.z, r0.w}, {r1.x, r1.y, r1.z, r1.w}};
    T.t = tok ? t : 0;
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
#if !TK_EXPAND_LDS_H
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int n0 = 32 * ks + 8 * kb;
        T.hop[tt][ks] = (tok && n0 < RP) ? ld16(hrow + (int64_t)(slot0 + 16 * tt + li) * RP + n0) : zero4();
      }
#endif
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        T.rows[tt][v] = (unsigned)rr[tt][v] < row_limit ? rr[tt][v] : -1;
        T.y[tt][v] = T.rows[tt][v] >= 0 ? ld16_nt(dst + (int64_t)T.rows[tt][v] * a.ld_dst) : zero4();
      }
    }
  };
  uint4 bq[8][NKS];
  int r = 0;
  auto load_weights = [&](int g) {  // this wave's block of W2 for group g
    r = CLS ? class_rank(a.rank[g], a.rank_lo, RP) : min(a.rank[g], RP);
    const bf16_t* W2 = group_weight<bf16_t>(a.w_expand, a.w_expand_base, a.expand_group_stride, g);
#pragma unroll
    for (int q = 0; q < 8; ++q)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int n0 = 32 * ks + 8 * kb;
        bq[q][ks] = n0 < r ? keep_first(ld16(W2 + (int64_t)(c0 + 8 * li + q) * a.ld_expand + n0), r - n0) : zero4();
      }
  };
  auto consume = [&](const Tile& T) {
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
#if TK_EXPAND_LDS_H
      uint4 hop[NKS];
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)
        hop[ks] = 32 * ks + 8 * kb < RP ? ld16(h_s + (T.t * kTileRows + 16 * tt + li) * HS + 32 * ks + 8 * kb) : zero4();
#endif
      f32x4 d[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        d[q] = f32x4{0.f, 0.f, 0.f, 0.f};
#if TK_EXPAND_LDS_H
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) d[q] = mfma16(hop[ks], bq[q][ks], d[q]);
#else
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) d[q] = mfma16(T.hop[tt][ks], bq[q][ks], d[q]);
#endif
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        if (T.rows[tt][v] < 0) continue;
        const uint4 yy = T.y[tt][v];
        uint4 o;
        o.x = pack_bf16(bf16_lo(yy.x) + d[0][v], bf16_hi(yy.x) + d[1][v]);
        o.y = pack_bf16(bf16_lo(yy.y) + d[2][v], bf16_hi(yy.y) + d[3][v]);
        o.z = pack_bf16(bf16_lo(yy.z) + d[4][v], bf16_hi(yy.z) + d[5][v]);
        o.w = pack_bf16(bf16_lo(yy.w) + d[6][v], bf16_hi(yy.w) + d[7][v]);
        st16_nt(dst + (int64_t)T.rows[tt][v] * a.ld_dst, o);
      }
    }
  };
  // tiles past the last one of the table carry -1 and come last
  bool uniform = true;
#pragma unroll
  for (int t = 1; t < TPI; ++t) uniform = uniform && (gt[t] == gt[0] || gt[t] < 0);
  Tile A, B;
  if (uniform) {  // the usual case: one group, one block of W2, loads pipelined over the tiles
    if (gt[0] < 0) return;
    int nv = 0;
#pragma unroll
    for (int t = 0; t < TPI; ++t) nv += gt[t] >= 0;
    load_weights(gt[0]);
    if (r <= 0) return;  // adapter not live on this layer
    issue(0, A);
    for (int t = 0; t < nv; t += 2) {
      issue(t + 1 < nv ? t + 1 : nt, B);
      consume(A);
      if (t + 1 < nv) {
        issue(t + 2 < nv ? t + 2 : nt, A);
        consume(B);
      }
    }
    return;
  }
  for (int t = 0; t < nt; ++t) {  // a group boundary inside the item: tile by tile
    if (gt[t] < 0) continue;
    load_weights(gt[t]);
    if (r <= 0) continue;
    issue(t, A);
    consume(A);
  }
}

// 8 x 8 block of bf16 transposed inside a lane: in[i] holds 8 consecutive elements of row i, out[q] the 8 rows'
// q-th elements (v_perm_b32 picks the low or the high halves of a register pair).
__device__ inline void transpose8x8(const uint4 (&in)[8], uint4 (&out)[8]) {
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const int d = q >> 1;
    const uint32_t sel = (q & 1) ? 0x07060302u : 0x05040100u;
    uint32_t e[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t w[4] = {in[i].x, in[i].y, in[i].z, in[i].w};
      e[i] = w[d];
    }
    out[q].x = __builtin_amdgcn_perm(e[1], e[0], sel);
    out[q].y = __builtin_amdgcn_perm(e[3], e[2], sel);
    out[q].z = __builtin_amdgcn_perm(e[5], e[4], sel);
    out[q].w = __builtin_amdgcn_perm(e[7], e[6], sel);
  }
}

// Eight consecutive weights as bf16, from a bf16 or an fp32 matrix (element index e, a multiple of 8 for the
// vector form; fp32 is rounded to nearest even).
__device__ inline uint4 load8_weights(const void* base, int64_t e, bool f32) {
  if (!f32) return ld16((const bf16_t*)base + e);
  const float4 lo = *reinterpret_cast<const float4*>((const float*)base + e);
  const float4 hi = *reinterpret_cast<const float4*>((const float*)base + e + 4);
  return make_uint4(pack_bf16(lo.x, lo.y), pack_bf16(lo.z, lo.w), pack_bf16(hi.x, hi.y), pack_bf16(hi.z, hi.w));
}
__device__ inline uint32_t load_weight(const void* base, int64_t e, bool f32) {
  return f32 ? (pack_bf16(((const float*)base)[e], 0.f) & 0xffffu) : (uint32_t)((const bf16_t*)base)[e];
}

// Transposed weight copies (see TransposeJob).  A work unit is an 8 x 8 block: eight 16-byte loads along the
// source's contiguous dimension, a transpose inside the lane, eight 16-byte stores along the copy's contiguous
// dimension; consecutive threads take neighbouring blocks so that a wave's accesses cover whole rows (128 bytes and
// more).  A source whose row stride or address rules out 16-byte loads is gathered element by element.
__device__ inline void transpose_weights_job(const TransposeJob& t, const int32_t* __restrict__ rank, int rpad,
                                             int64_t thread, int64_t threads) {
  const int m8 = t.out_features >> 3, n8 = rpad >> 3, k8 = t.in_features >> 3;
  const int64_t units_b = t.bT ? (int64_t)t.groups * m8 * n8 : 0;  // (g, m-octet, n-octet), n-octet fastest
  const int64_t units_a = (int64_t)t.groups * n8 * k8;              // (g, k-octet, n-octet), n-octet fastest
  const bool f32 = t.src_f32 != 0;
  const int ld_mask = f32 ? 3 : 7;  // row strides that keep every row 16-byte aligned
  for (int64_t u = thread; u < units_b + units_a; u += threads) {
    uint4 in[8], out[8];
    if (u < units_b) {
      // bT[g][n][m] = B_g[m][n]: rows m of B hold the rank index contiguously
      const int no = (int)(u % n8);
      const int64_t q = u / n8;
      const int mo = (int)(q % m8), g = (int)(q / m8);
      const int r = class_rank(rank[g], t.rank_lo, rpad);
      if (8 * no >= r && t.skip_dead) continue;
      const void* B = t.lora_B[g];
      const int64_t b0 = (int64_t)(8 * mo) * t.ldb + 8 * no;
      const bool vec = (t.ldb & ld_mask) == 0 && 8 * no + 8 <= t.ldb && (reinterpret_cast<uintptr_t>(B) & 15u) == 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (8 * no >= r) {
          in[i] = zero4();
        } else if (vec) {
          in[i] = keep_first(load8_weights(B, b0 + (int64_t)i * t.ldb, f32), r - 8 * no);
        } else {
          uint32_t e[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) e[j] = 8 * no + j < r ? load_weight(B, b0 + (int64_t)i * t.ldb + j, f32) : 0;
          in[i] = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
        }
      }
      transpose8x8(in, out);
      bf16_t* o = (bf16_t*)t.bT + ((int64_t)g * rpad + 8 * no) * t.out_features + 8 * mo;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (8 * no + j < r || !t.skip_dead) st16(o + (int64_t)j * t.out_features, out[j]);
    } else {
      // aT[g][k][n] = A_g[n][k]: rows n of A hold the input features contiguously
      // rank octet fastest: the threads that hold the octets of one column of A are neighbours, so a wave-wide
      // store covers whole rows of the copy (a row is rpad elements), and a wave-wide load still covers 128-byte
      // runs of A's rows (eight neighbouring column octets per rank octet)
      const int64_t v = u - units_b;
      const int no = (int)(v % n8);
      const int64_t q = v / n8;
      const int ko = (int)(q % k8), g = (int)(q / k8);
      const int r = class_rank(rank[g], t.rank_lo, rpad);
      if (8 * no >= r && t.skip_dead) continue;
      const void* A = t.lora_A[g];
      const int64_t a0 = (int64_t)(8 * no) * t.lda + 8 * ko;
      const bool vec = (t.lda & ld_mask) == 0 && (reinterpret_cast<uintptr_t>(A) & 15u) == 0;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (8 * no + i >= r) {
          in[i] = zero4();
        } else if (vec) {
          in[i] = load8_weights(A, a0 + (int64_t)i * t.lda, f32);
        } else {
          uint32_t e[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) e[j] = load_weight(A, a0 + (int64_t)i * t.lda + j, f32);
          in[i] = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
        }
      }
      transpose8x8(in, out);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = 8 * ko + j;  // column of A; which row of aT holds it:
        const int kd = t.swizzle_a ? ((k & ~127) | ((k & 7) << 4) | ((k >> 3) & 15)) : k;
        st16((bf16_t*)t.aT + ((int64_t)g * t.in_features + kd) * rpad + 8 * no, out[j]);
      }
    }
  }
}

// The transposed copies as a launch of their own (backward paths whose first kernel cannot carry them as a side job).
__global__ __launch_bounds__(256) void k_transpose_job(TransposeJob t, const int32_t* __restrict__ rank, int rpad) {
  transpose_weights_job(t, rank, rpad, (int64_t)blockIdx.x * 256 + threadIdx.x, (int64_t)gridDim.x * 256);
}

// ---------------------------------------------------------------------------
// Weight gradient: out_g[n][c] = sum over the rows of group g of hT[n][slot] * src[row(slot)][c].
//
// Work item = (chunk of one group, 128 source columns), one wave.  The wave walks all tiles of
// the chunk with an S-stage software pipeline: the source rows of tile t+S-1 are requested before tile t
// is consumed, so a wave has S-1 tiles (8 KB each) in flight; the chunk's row indices wait in LDS, where
// reading them does not have to wait for the tile loads in flight.  A grid of (chunks x 128-column
// blocks) is small next to the chip, so the depth of the pipeline, not the number of resident waves, is
// what keeps enough bytes in flight.  A lane loads 16 B of eight rows, transposes the 8x8 block in registers
// (v_perm_b32) and feeds it as the MFMA A operand with the rows as contraction index.  The result is
// staged in LDS in [n][column] order and leaves as whole 512-byte rows: into the chunk's slot of the
// partial buffer (groups that span several chunks; k_wgrad_reduce adds the chunks in order) or straight
// into the gradient (single-chunk groups).  No atomics: the result is bitwise repeatable.
//
// This one-wave form serves padded rank 16; above it two waves share the tiles (k_wgrad_coop below).
// ---------------------------------------------------------------------------
template <int NB, int S>
__global__ __launch_bounds__(64) void k_wgrad_pipe(WgradArgs a, const ChunkInfo* __restrict__ chunks,
                                                        const int32_t* __restrict__ slot_rows) {
  constexpr int OS = kWgradStageStride;
  __shared__ __attribute__((aligned(16))) float lds[16 * NB * OS];
  extern __shared__ __attribute__((aligned(16))) int32_t rows_s[];  // the chunk's row indices
  const int tid = threadIdx.x, lane = tid & 63, li = lane & 15, kb = lane >> 4;
  if ((int)blockIdx.y < a.tr.y_blocks) {  // side job: the first rows of the grid transpose the adapter weights
    transpose_weights_job(a.tr, a.rank, a.rpad, ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * 64 + tid,
                          (int64_t)a.tr.y_blocks * gridDim.x * 64);
    return;
  }
  // column block fastest: blocks that run together read neighbouring pieces of the same rows
  const int c0 = blockIdx.x * 128;
  const int cidx = work_item(a.wl_chunks, blockIdx.y - a.tr.y_blocks);
  if (cidx < 0) return;  // past the end of this rank class's list
  const ChunkInfo ci = checked_chunk(chunks[cidx], a.tb);
  const int g = ci.group;
  if (g < 0) return;
  const int r = class_rank(a.rank[g], a.rank_lo, 16 * NB);
  if (r <= 0) return;
  const int nt = ci.ntiles;
  for (int i = tid; i < nt * kTileRows; i += 64) rows_s[i] = slot_rows[ci.tile0 * kTileRows + i];
  __syncthreads();

  const bf16_t* src = (const bf16_t*)a.src + c0 + 8 * li;
  const bf16_t* hT = (const bf16_t*)a.hT + (int64_t)li * a.ldh + (int64_t)ci.tile0 * kTileRows + 8 * kb;
  f32x4 acc[8][NB];
#pragma unroll
  for (int q = 0; q < 8; ++q)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[q][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // The loop body below is straight-line code: every load is unconditional (tiles past the end re-read the
  // last tile, padding slots read row 0) and what must not count is zeroed when it is consumed.  With no
  // branch between a load and its use the compiler can wait for exactly the loads it needs and leave the
  // younger ones in flight.
  struct Tile {
    uint4 x[8];
    uint4 h[NB];
    uint32_t live;  // bit q: row q of this lane is a real row of a tile inside the chunk
  };
  auto issue = [&](int t, Tile& T) {
    const int tc = min(t, nt - 1);
    const int4 ra = *reinterpret_cast<const int4*>(rows_s + tc * kTileRows + 8 * kb);
    const int4 rb = *reinterpret_cast<const int4*>(rows_s + tc * kTileRows + 8 * kb + 4);
    const int rows[8] = {ra.x, ra.y, ra.z, ra.w, rb.x, rb.y, rb.z, rb.w};
    T.live = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int row = checked_row(rows[q], a.tb);
      T.x[q] = ld16(src + (int64_t)max(row, 0) * a.ld_src);
      T.live |= (t < nt && row >= 0) ? (1u << q) : 0u;
    }
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) T.h[nb] = ld16(hT + (int64_t)(16 * nb) * a.ldh + tc * kTileRows);
  };
  auto consume = [&](const Tile& T) {
    // 8x8 transpose inside the lane: tr holds column q of the 8 rows
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int d = q >> 1;
      const uint32_t sel = (q & 1) ? 0x07060302u : 0x05040100u;
      uint32_t e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t wsrc[4] = {T.x[i].x, T.x[i].y, T.x[i].z, T.x[i].w};
        e[i] = (T.live >> i) & 1u ? wsrc[d] : 0u;
      }
      uint4 tr;
      tr.x = __builtin_amdgcn_perm(e[1], e[0], sel);
      tr.y = __builtin_amdgcn_perm(e[3], e[2], sel);
      tr.z = __builtin_amdgcn_perm(e[5], e[4], sel);
      tr.w = __builtin_amdgcn_perm(e[7], e[6], sel);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[q][nb] = mfma16(tr, T.h[nb], acc[q][nb]);
    }
  };
  Tile T[S];
#pragma unroll
  for (int i = 0; i < S - 1; ++i) issue(i, T[i]);
  int t = 0;
  for (; t + S <= nt; t += S) {  // every tile consumed in here exists (the youngest requests may lie past the end)
#pragma unroll
    for (int i = 0; i < S; ++i) {
      issue(t + i + S - 1, T[(i + S - 1) % S]);
      consume(T[i]);
    }
  }
  // drain: fewer than S tiles are left, all requested already (tiles past the end count as zeros)
#pragma unroll
  for (int i = 0; i < S - 1; ++i) consume(T[i]);
  wgrad_store<NB>(acc, lds, a, ci, g, r, c0, lane);
}

// ---------------------------------------------------------------------------
// Weight gradient at padded rank 32 and 64: (chunk, 128 columns), two waves, each owning half of the rank
// indices and both needing every tile of the source (one wave with all of them would hold 64 or 128
// accumulator registers next to its tiles in flight: measured 49 against 41 us at rank 32, one wave per SIMD
// at rank 64).  Two independent readers of a tile drift apart and the later one misses the CU's cache
// (measured at rank 64: 1.66 x the source bytes fetched from memory), so here the tile crosses the
// memory system once: each wave requests half of it (4 of the 8 rows of every lane's 8 x 8 block), S - 1
// tiles ahead, the halves meet in a double-buffered LDS tile behind an LDS-only barrier (global loads stay
// in flight), and every wave reads the whole tile back in the operand layout.  Padding rows are zeroed when
// they are written to LDS.  One barrier per tile: a wave overwrites a buffer two tiles later, after the
// barrier that every reader of it has passed.
// ---------------------------------------------------------------------------
// PAIRS: pairs of waves per block (1 or 2).  Two pairs take neighbouring column blocks of the same chunk: they load
// the same h operands at about the same time, so the second pair's come from the CU's cache instead of from L2
// (every 128-column block of a chunk re-reads the chunk's h: a third of this kernel's L2 reads at rank 64).
template <int NB, int S, int PAIRS = 1>
__device__ __forceinline__ void wgrad_coop_body(const WgradArgs& a, const ChunkInfo* __restrict__ chunks,
                                                const int32_t* __restrict__ slot_rows, int bx, int by, int nx) {
  constexpr int RS = 2, NBW = NB / 2;
  constexpr int OS = kWgradStageStride;
  constexpr int XS = 136;  // row stride of a staged tile in bf16 (272 B)
  // the tile buffers are dead when the result is staged: one array serves both
  constexpr int kLdsFloats = 16 * NB * OS > kTileRows * XS ? 16 * NB * OS : kTileRows * XS;  // >= two staged bf16 tiles
  __shared__ __attribute__((aligned(16))) float lds_all[PAIRS * kLdsFloats];
  float* const lds = lds_all + (PAIRS > 1 ? (threadIdx.x >> 7) * kLdsFloats : 0);
  extern __shared__ __attribute__((aligned(16))) int32_t rows_s[];  // the chunk's row indices (same for both pairs)
  const int tid = threadIdx.x & 127, lane = tid & 63, li = lane & 15, kb = lane >> 4, rs = tid >> 6;
  if (by < a.tr.y_blocks) {  // side job: the first rows of the grid transpose the adapter weights
    transpose_weights_job(a.tr, a.rank, a.rpad, ((int64_t)by * nx + bx) * (RS * 64) + tid,
                          (int64_t)a.tr.y_blocks * nx * (RS * 64));
    return;
  }
  const int c0 = bx * 128;
  const int cidx = work_item(a.wl_chunks, by - a.tr.y_blocks);
  if (cidx < 0) return;  // past the end of this rank class's list
  const ChunkInfo ci = checked_chunk(chunks[cidx], a.tb);
  const int g = ci.group;
  if (g < 0) return;
  int nt = ci.ntiles;
  if (a.pair_chunks) {  // (the neighbours' entries do not depend on ci: three loads side by side)
    const ChunkInfo none{-1, 0, 0, -1};
    const ChunkInfo before = cidx > 0 ? checked_chunk(chunks[cidx - 1], a.tb) : none;
    const ChunkInfo after = cidx + 1 < a.tb.max_chunks ? checked_chunk(chunks[cidx + 1], a.tb) : none;
    if (chunk_follows(before, ci)) return;  // the block of the chunk in front takes this one's tiles
    if (chunk_follows(ci, after)) nt += after.ntiles;
  }
  const int r = class_rank(a.rank[g], a.rank_lo, 16 * NB);
  if (r <= 0) return;
  for (int i = tid; i < nt * kTileRows; i += RS * 64) rows_s[i] = slot_rows[ci.tile0 * kTileRows + i];
  __syncthreads();
  const int n_base = rs * NBW * 16;   // first rank index of this wave
  const bool mine = r > n_base;       // a wave without live rank indices still carries its half of every tile

  bf16_t* tiles = reinterpret_cast<bf16_t*>(lds);
  const bf16_t* src = (const bf16_t*)a.src + c0 + 8 * li;
  const bf16_t* hT = (const bf16_t*)a.hT + (int64_t)(n_base + li) * a.ldh + (int64_t)ci.tile0 * kTileRows + 8 * kb;
  f32x4 acc[8][NBW];
#pragma unroll
  for (int q = 0; q < 8; ++q)
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) acc[q][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  struct Piece {
    uint4 x[4];      // rows 8 kb + 4 rs + i of the tile, columns 8 li .. 8 li + 7
    uint4 h[NBW];
    uint32_t live;
  };
  auto issue = [&](int t, Piece& P) {
    const int tc = min(t, nt - 1);
    const int4 rr = *reinterpret_cast<const int4*>(rows_s + tc * kTileRows + 8 * kb + 4 * rs);
    const int rows[4] = {rr.x, rr.y, rr.z, rr.w};
    P.live = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = checked_row(rows[i], a.tb);
      P.x[i] = ld16(src + (int64_t)max(row, 0) * a.ld_src);
      P.live |= row >= 0 ? (1u << i) : 0u;
    }
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) P.h[nb] = ld16(hT + (int64_t)(16 * nb) * a.ldh + tc * kTileRows);
  };
  auto consume = [&](int t, const Piece& P) {
    bf16_t* buf = tiles + (t & 1) * (kTileRows * XS);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      st16(buf + (8 * kb + 4 * rs + i) * XS + 8 * li, (P.live >> i) & 1u ? P.x[i] : zero4());
    lds_barrier();
    if (!mine) return;
    uint4 x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = ld16(buf + (8 * kb + i) * XS + 8 * li);
    // 8x8 transpose inside the lane: tr holds column q of the 8 rows
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
      uint4 tr;
      tr.x = __builtin_amdgcn_perm(e[1], e[0], sel);
      tr.y = __builtin_amdgcn_perm(e[3], e[2], sel);
      tr.z = __builtin_amdgcn_perm(e[5], e[4], sel);
      tr.w = __builtin_amdgcn_perm(e[7], e[6], sel);
#pragma unroll
      for (int nb = 0; nb < NBW; ++nb) acc[q][nb] = mfma16(tr, P.h[nb], acc[q][nb]);
    }
  };
  Piece T[S];
#pragma unroll
  for (int i = 0; i < S - 1; ++i) issue(i, T[i]);
  int t = 0;
  for (; t + S <= nt; t += S) {  // every tile consumed in here exists (the youngest requests may lie past the end)
#pragma unroll
    for (int i = 0; i < S; ++i) {
      issue(t + i + S - 1, T[(i + S - 1) % S]);
      consume(t + i, T[i]);
    }
  }
  // fewer than S tiles are left, all of them requested already; both waves take the same trips (barriers inside)
#pragma unroll
  for (int i = 0; i < S - 1; ++i)
    if (t + i < nt) consume(t + i, T[i]);
  __syncthreads();  // the last tile has been read everywhere: its buffer becomes the staging area
  if (mine) wgrad_store<NBW>(acc, lds + n_base * OS, a, ci, g, r, c0, lane, n_base);
}

template <int NB, int S, int PAIRS>
__global__ __launch_bounds__(128 * PAIRS) void k_wgrad_coop(WgradArgs a, const ChunkInfo* __restrict__ chunks,
                                                              const int32_t* __restrict__ slot_rows) {
  wgrad_coop_body<NB, S, PAIRS>(a, chunks, slot_rows, blockIdx.x * PAIRS + (PAIRS > 1 ? threadIdx.x >> 7 : 0), blockIdx.y,
                                gridDim.x * PAIRS);
}

// The same contraction for up to kMaxShared projections that read the same source (dA_p = dh_p^T x for the
// projections of one input): one launch, the bodies of k_wgrad_coop, every tile of the source crossing memory
// once (see shared_source_item).  Work item = (chunk, 128 columns), column block fastest.
template <int NB, int S>
__global__ __launch_bounds__(128) void k_wgrad_coop_multi(SharedWgradArgs jobs, int items, int nx,
                                                            const ChunkInfo* __restrict__ chunks,
                                                            const int32_t* __restrict__ slot_rows) {
  int p, item;
  shared_source_item(blockIdx.x, jobs.nproj, p, item);
  if (item >= items) return;
  wgrad_coop_body<NB, S>(jobs.w[p], chunks, slot_rows, item % nx, item / nx, nx);
}

// ---------------------------------------------------------------------------
// Backward, both uses of dy in one pass (rank <= 16 NB, NB = 1 or 2; width a multiple of 512): a block of four waves owns
// (chunk of one group, 512 columns), wave w the columns [128 w, 128 w + 128) of it.
// Per tile a wave loads its 32 x 128 piece once, in the weight-gradient layout (a lane holds 8 rows x 8
// columns), and uses it twice:
//   dB:  the piece, transposed in registers, is the MFMA A operand with the rows as contraction index,
//        accumulated over the chunk's tiles exactly like k_wgrad_pipe does;
//   dh:  the piece goes through a per-wave LDS buffer to come back in the row-major operand layout and
//        is multiplied with the wave's 128 x rank block of B (loaded once per chunk, straight from the
//        adapter's [out][r] layout); the four waves' partial dh[32][rank] meet in LDS after a block
//        barrier and one of them writes the sum as slice `blockIdx.x` of the split-shrink buffer, which
//        k_shrink_finish turns into dh like after a separate shrink.
// dy crosses the memory system once instead of twice.  Sums are formed in a fixed order.
// ---------------------------------------------------------------------------
template <int NB>
__device__ __forceinline__ void dy_fused_body(const WgradArgs& a, const void* const* __restrict__ lora_B, int64_t ldb,
                                              float* __restrict__ hpart, int kslices,
                                              const ChunkInfo* __restrict__ chunks,
                                              const int32_t* __restrict__ slot_rows, int bx, int by, int x_blocks) {
  constexpr int RP = 16 * NB;
  constexpr int SS = 136;     // row stride of the staged piece in bf16 (272 B)
  constexpr int PR = RP + 1;  // row stride of the partial dh in floats
  extern __shared__ int32_t rows_s[];  // the chunk's row indices (chunk_tiles x 32)
  __shared__ __attribute__((aligned(16))) bf16_t stage[4][kTileRows * SS];
  __shared__ float part[2][4][kTileRows * PR];
  static_assert(sizeof(bf16_t) * kTileRows * SS >= sizeof(float) * 16 * kWgradStageStride, "stage holds a dB block too");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  if (by < a.tr.y_blocks) {  // side job: the first rows of the grid transpose the adapter weights
    transpose_weights_job(a.tr, a.rank, a.rpad, ((int64_t)by * x_blocks + bx) * 256 + tid,
                          (int64_t)a.tr.y_blocks * x_blocks * 256);
    return;
  }
  const int cidx = work_item(a.wl_chunks, by - a.tr.y_blocks);
  if (cidx < 0) return;  // past the end of this rank class's list
  const ChunkInfo ci = checked_chunk(chunks[cidx], a.tb);
  const int g = ci.group;
  if (g < 0) return;
  const int r = class_rank(a.rank[g], a.rank_lo, RP);
  if (r <= 0) return;
  const int slab = bx;
  const int c0 = slab * 512 + wave * 128;
  const int nt = ci.ntiles;
  for (int i = tid; i < nt * kTileRows; i += 256) rows_s[i] = slot_rows[ci.tile0 * kTileRows + i];
  // this wave's block of B as MFMA B operand: lane (n = 16 nb + li, kb) holds B[c0 + 32 s + 8 kb + i][n], i = 0..7
  uint4 wB[NB][4];
  const void* Bsrc = lora_B[g];
  const bool b_f32 = a.grad_f32 != 0;  // fp32 adapters: converted as they are loaded
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int n = 16 * nb + li;
    const int64_t b0 = (int64_t)(c0 + 8 * kb) * ldb + (n < r ? n : 0);
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) {
      uint32_t e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i)  // (the address is valid for every lane: loads first, masks after)
        e[i] = load_weight(Bsrc, b0 + (int64_t)(32 * s4 + i) * ldb, b_f32);
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = n < r ? e[i] : 0;
      wB[nb][s4] = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16));
    }
  }
  __syncthreads();

  const bf16_t* src = (const bf16_t*)a.src + c0 + 8 * li;
  const bf16_t* hT = (const bf16_t*)a.hT + (int64_t)li * a.ldh + (int64_t)ci.tile0 * kTileRows + 8 * kb;
  bf16_t* my_stage = stage[wave];
  f32x4 acc[8][NB];
#pragma unroll
  for (int q = 0; q < 8; ++q)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[q][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // loads are unconditional (tiles past the end re-read the last one, padding slots read row 0) and what
  // must not count is zeroed when it is consumed: no branch between a load and its use
  auto issue = [&](int t, uint4 (&x)[8], uint4 (&h)[NB], uint32_t& live) {
    const int tc = min(t, nt - 1);
    const int4 ra = *reinterpret_cast<const int4*>(rows_s + tc * kTileRows + 8 * kb);
    const int4 rb = *reinterpret_cast<const int4*>(rows_s + tc * kTileRows + 8 * kb + 4);
    const int rows[8] = {ra.x, ra.y, ra.z, ra.w, rb.x, rb.y, rb.z, rb.w};
    live = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int row = checked_row(rows[q], a.tb);
      x[q] = ld16(src + (int64_t)max(row, 0) * a.ld_src);
      live |= (t < nt && row >= 0) ? (1u << q) : 0u;
    }
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) h[nb] = ld16(hT + (int64_t)(16 * nb) * a.ldh + tc * kTileRows);
  };
  auto consume = [&](int t, uint4 (&x)[8], const uint4 (&h)[NB], uint32_t live) {
#pragma unroll
    for (int q = 0; q < 8; ++q)
      if (!((live >> q) & 1u)) x[q] = zero4();
    // the piece in row-major order for the dh product
#pragma unroll
    for (int q = 0; q < 8; ++q) st16(my_stage + (8 * kb + q) * SS + 8 * li, x[q]);
    // dB: 8x8 transpose inside the lane, rows become the contraction index
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
      uint4 tr;
      tr.x = __builtin_amdgcn_perm(e[1], e[0], sel);
      tr.y = __builtin_amdgcn_perm(e[3], e[2], sel);
      tr.z = __builtin_amdgcn_perm(e[5], e[4], sel);
      tr.w = __builtin_amdgcn_perm(e[7], e[6], sel);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[q][nb] = mfma16(tr, h[nb], acc[q][nb]);
    }
  };
  // dh of tile t from the staged piece: partial over this wave's 128 columns (LDS operations of one wave complete
  // in order); needs no register of the tile any more
  auto consume_dh = [&](int t) {
    float* mine = part[t & 1][wave];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      f32x4 d[NB];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) d[nb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        const uint4 piece = ld16(my_stage + (16 * tt + li) * SS + 32 * s4 + 8 * kb);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) d[nb] = mfma16(piece, wB[nb][s4], d[nb]);
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int v = 0; v < 4; ++v) mine[(16 * tt + 4 * kb + v) * PR + 16 * nb + li] = d[nb][v];
    }
    lds_barrier();
    if (wave == (t & 3)) {
      float* o = hpart + ((int64_t)(ci.tile0 + t) * kslices + slab) * (kTileRows * RP);
#pragma unroll
      for (int i = 0; i < 8 * NB; ++i) {
        const int idx = lane + 64 * i, row = idx / RP, n = idx % RP;
        float sum = part[t & 1][0][row * PR + n];
        sum += part[t & 1][1][row * PR + n];
        sum += part[t & 1][2][row * PR + n];
        sum += part[t & 1][3][row * PR + n];
        o[idx] = sum;
      }
    }
  };

  constexpr int S = NB == 1 ? TK_DY_STAGES : TK_DY_STAGES2;  // software pipeline: S - 1 tiles in flight while one is consumed
  struct Tile {
    uint4 x[8];
    uint4 h[NB];
    uint32_t live;
  };
  Tile T[S];
  if constexpr (S == 1) {
    // one tile in registers: its successor is requested as soon as the dB products have used it up, and is in
    // flight during the dh half of the iteration
    issue(0, T[0].x, T[0].h, T[0].live);
    for (int t = 0; t < nt; ++t) {
      consume(t, T[0].x, T[0].h, T[0].live);
      issue(t + 1, T[0].x, T[0].h, T[0].live);
      consume_dh(t);
    }
  } else {
#pragma unroll
    for (int i = 0; i < S - 1; ++i) issue(i, T[i].x, T[i].h, T[i].live);
    int t = 0;
    for (; t + S <= nt; t += S) {  // every tile consumed in here exists (the youngest requests may lie past the end)
#pragma unroll
      for (int i = 0; i < S; ++i) {
        Tile& Y = T[(i + S - 1) % S];
        issue(t + i + S - 1, Y.x, Y.h, Y.live);
        consume(t + i, T[i].x, T[i].h, T[i].live);
        consume_dh(t + i);
      }
    }
    // fewer than S tiles are left, all of them requested already
#pragma unroll
    for (int i = 0; i < S - 1; ++i)
      if (t + i < nt) {
        consume(t + i, T[i].x, T[i].h, T[i].live);
        consume_dh(t + i);
      }
  }
  // every wave has its own 128 columns of dB; they leave 16 rank indices at a time through the wave's stage
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    if (16 * nb >= r) break;
    f32x4 one[8][1];
#pragma unroll
    for (int q = 0; q < 8; ++q) one[q][0] = acc[q][nb];
    wgrad_store<1>(one, reinterpret_cast<float*>(my_stage), a, ci, g, r, c0, lane, 16 * nb);
  }
}

template <int NB>
__global__ __launch_bounds__(256) void k_dy_fused(WgradArgs a, const void* const* __restrict__ lora_B, int64_t ldb,
                                                  float* __restrict__ hpart, int kslices,
                                                  const ChunkInfo* __restrict__ chunks,
                                                  const int32_t* __restrict__ slot_rows) {
  dy_fused_body<NB>(a, lora_B, ldb, hpart, kslices, chunks, slot_rows, blockIdx.x, blockIdx.y, gridDim.x);
}

// Up to kMaxShared projections in one launch: a narrow projection alone has too few (chunk, 512 columns)
// blocks to fill the chip.  The jobs' column slabs lie side by side along blockIdx.x, so that the blocks of
// all projections are dispatched interleaved and run next to each other.
__global__ __launch_bounds__(256) void k_dy_fused_multi(DyFusedJobs jobs, const ChunkInfo* __restrict__ chunks,
                                                        const int32_t* __restrict__ slot_rows, int max_chunks) {
  int p = 0;
#pragma unroll
  for (int i = 1; i < kMaxShared; ++i) p += (i < jobs.n && (int)blockIdx.x >= jobs.x_first[i]) ? 1 : 0;
  const DyFusedJob& j = jobs.j[p];
  if ((int)blockIdx.y >= j.a.tr.y_blocks + max_chunks) return;
  dy_fused_body<1>(j.a, j.lora_B, j.ldb, j.hpart, j.kslices, chunks, slot_rows, blockIdx.x - jobs.x_first[p],
                   blockIdx.y, j.x_blocks);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int NB>
void launch_pass(const PassArgs& a, const SegView& seg, const SegLayout& L, int phases, hipStream_t s) {
  bf16_t* hrow = (bf16_t*)a.hT + (int64_t)a.rpad * a.ldh;  // second half of the h buffer
  const int32_t* rows = seg.slot_table(a.map_rows);
  constexpr int NW = NB == 1 ? 1 : (NB == 2 ? 2 : 4);  // shrink_waves(16 * NB)
  if (phases & 1) {
    if (NB > 1 && a.quad_steps > 0)  // see shrink_plan
      hipLaunchKernelGGL((k_shrink_quad<NB>), dim3((unsigned)(ceil_div(L.max_tiles, 8) * a.kslices)), dim3(256), 0, s,
                         a, seg.tile_group, rows, (int)L.max_tiles);
    else
      hipLaunchKernelGGL((k_shrink_pair<NB, NW>), dim3((unsigned)(ceil_div(L.max_tiles, 2) * a.kslices)),
                         dim3(NW * 64), 0, s, a, hrow, seg.tile_group, rows, (int)L.max_tiles);
  }
  if ((phases & 5) && a.kslices > 1)
    hipLaunchKernelGGL((k_shrink_finish<NB>), dim3((unsigned)L.max_tiles), dim3(256), 0, s, a, hrow, seg.tile_group,
                       rows);
  if (!a.dst || !(phases & 2)) return;
  const int64_t ngroups = a.width_dst >> 7;
  if constexpr (NB > 1) {
    constexpr int TPI = 4;
    const int64_t blocks = ceil_div(L.max_tiles, TPI) * ceil_div(ngroups, 4);
    const auto kernel = a.wl_sets.ids ? k_expand_multi<NB, TPI, true> : k_expand_multi<NB, TPI, false>;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, s, a, hrow, seg.tile_group, rows,
                       seg.set_walk(a.map_rows), seg.header, seg.round_moved,
                       (int)std::min<int64_t>(L.sort_blocks, 64), (int)L.max_tiles);
  } else {
    const int64_t items = L.max_tiles * ngroups;
    hipLaunchKernelGGL((k_expand_mfma<NB>), dim3((unsigned)ceil_div(items, 4)), dim3(256), 0, s, a, hrow,
                       seg.tile_group, rows, seg.tile_walk(a.map_rows), (int)items);
  }
}

template <int NB, int S>
void launch_wgrad_pipe(const WgradArgs& a0, const SegView& seg, const SegLayout& L, hipStream_t s) {
  WgradArgs a = a0;
  a.tr.y_blocks = 0;
  if (a.tr.aT) {  // about four 16-byte outputs per thread of the side job
    const int64_t units = (int64_t)a.tr.groups * a.rpad * ((a.tr.out_features + a.tr.in_features) / 64);
    a.tr.y_blocks = (int)std::min<int64_t>(64, std::max<int64_t>(1, units / (2 * (a.width / 128) * 64)));
  }
  const dim3 grid((unsigned)(a.width / 128), (unsigned)(L.max_chunks + a.tr.y_blocks));
  const size_t dyn = (size_t)L.chunk_tiles * kTileRows * sizeof(int32_t);  // a chunk's row indices
  hipLaunchKernelGGL((k_wgrad_pipe<NB, S>), grid, dim3(64), dyn, s, a, seg.chunks,
                     seg.slot_table(a.map_rows));
}

template <int NB>
void launch_wgrad_coop(const WgradArgs& a0, const SegView& seg, const SegLayout& L, hipStream_t s) {
  constexpr int S = TK_COOP_STAGES;
  WgradArgs a = a0;
  a.tr.y_blocks = 0;
  if (a.tr.aT) {
    const int64_t units = (int64_t)a.tr.groups * a.rpad * ((a.tr.out_features + a.tr.in_features) / 64);
    a.tr.y_blocks = (int)std::min<int64_t>(64, std::max<int64_t>(1, units / (2 * (a.width / 128) * 128)));
  }
  const int nx = a.width / 128;
  const size_t dyn = (size_t)L.chunk_tiles * kTileRows * sizeof(int32_t) * (a.pair_chunks ? 2 : 1);
  // Two pairs per block only where that still leaves every CU several blocks (the grid counts every chunk slot of
  // the table): measured at config 3 (65 chunk slots x 112 / 32 column blocks) 2.4 % of the step; at config 5's
  // q projection (41 x 32) the coarser blocks balance worse over the CUs and cost 13 %.
  if (TK_COOP_PAIRS == 2 && nx % 2 == 0 && (int64_t)nx * L.max_chunks >= 8 * 256) {
    const dim3 grid((unsigned)(nx / 2), (unsigned)(L.max_chunks + a.tr.y_blocks));
    hipLaunchKernelGGL((k_wgrad_coop<NB, S, 2>), grid, dim3(256), dyn, s, a, seg.chunks, seg.slot_table(a.map_rows));
  } else {
    const dim3 grid((unsigned)nx, (unsigned)(L.max_chunks + a.tr.y_blocks));
    hipLaunchKernelGGL((k_wgrad_coop<NB, S, 1>), grid, dim3(128), dyn, s, a, seg.chunks, seg.slot_table(a.map_rows));
  }
}

}  // namespace

bool dy_fused_supported(const WgradArgs& a, int kslices) {
  return (a.rpad == 16 || a.rpad == 32) && a.width % 512 == 0 && kslices >= 2 && kslices == a.width / 512 &&
         wgrad_mfma_supported(a);
}

int launch_dy_fused(const WgradArgs& a0, const void* const* lora_B, int64_t ldb, float* hpart, int kslices,
                    const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  WgradArgs a = a0;
  a.tr.y_blocks = 0;
  if (a.tr.aT) {
    const int64_t units = (int64_t)a.tr.groups * a.rpad * ((a.tr.bT ? a.tr.out_features : 0) + a.tr.in_features) / 64;
    a.tr.y_blocks = (int)std::min<int64_t>(64, std::max<int64_t>(1, units / (2 * (a.width / 512) * 256)));
  }
  const dim3 grid((unsigned)(a.width / 512), (unsigned)(L.max_chunks + a.tr.y_blocks));
  const size_t dyn = (size_t)L.chunk_tiles * kTileRows * sizeof(int32_t);  // a chunk's row indices
  if (a.rpad == 16)
    hipLaunchKernelGGL(k_dy_fused<1>, grid, dim3(256), dyn, s, a, lora_B, ldb, hpart, kslices, seg.chunks,
                       seg.slot_table(a.map_rows));
  else
    hipLaunchKernelGGL(k_dy_fused<2>, grid, dim3(256), dyn, s, a, lora_B, ldb, hpart, kslices, seg.chunks,
                       seg.slot_table(a.map_rows));
  return check_launch();
}

int launch_dy_fused_multi(const DyFusedJob* jobs, int n, const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0 || n == 0) return TK_OK;
  DyFusedJobs J{};
  J.n = n;
  int gy = 0;
  for (int p = 0; p < n; ++p) {
    DyFusedJob& j = J.j[p];
    j = jobs[p];
    j.x_blocks = j.a.width / 512;
    j.a.tr.y_blocks = 0;
    if (j.a.tr.aT) {
      const int64_t units =
          (int64_t)j.a.tr.groups * j.a.rpad * ((j.a.tr.bT ? j.a.tr.out_features : 0) + j.a.tr.in_features) / 64;
      j.a.tr.y_blocks = (int)std::min<int64_t>(64, std::max<int64_t>(1, units / (2 * j.x_blocks * 256)));
    }
    J.x_first[p + 1] = J.x_first[p] + j.x_blocks;
    gy = std::max(gy, (int)L.max_chunks + j.a.tr.y_blocks);
  }
  const size_t dyn = (size_t)L.chunk_tiles * kTileRows * sizeof(int32_t);
  hipLaunchKernelGGL(k_dy_fused_multi, dim3((unsigned)J.x_first[n], (unsigned)gy), dim3(256), dyn, s, J, seg.chunks,
                     seg.slot_table(J.j[0].a.map_rows), (int)L.max_chunks);
  return check_launch();
}

// Finish and / or flat expand of several projections of padded rank 16 (phases: 4 finish, 2 expand).
int launch_pass_multi(const PassArgs* a, int n, const SegView& seg, const SegLayout& L, int phases, hipStream_t s) {
  if (L.rows == 0 || n == 0) return TK_OK;
  PassJobs J{};
  int64_t widest = 0;
  for (int p = 0; p < n; ++p) {
    J.p[p] = a[p];
    widest = std::max<int64_t>(widest, a[p].width_dst >> 7);
  }
  const int32_t* rows = seg.slot_table(a[0].map_rows);
  if (phases & 4)
    hipLaunchKernelGGL(k_shrink_finish_multi, dim3((unsigned)L.max_tiles, (unsigned)n), dim3(256), 0, s, J,
                       seg.tile_group, rows);
  if (phases & 2)
    hipLaunchKernelGGL(k_expand_mfma_multi, dim3((unsigned)ceil_div(L.max_tiles * widest, 4), (unsigned)n), dim3(256), 0,
                       s, J, seg.tile_group, rows, seg.tile_walk(a[0].map_rows), (int)L.max_tiles);
  return check_launch();
}

// B^T / A^T copies for the MFMA shrink and expand of a backward pass (bf16, out_features a multiple of 8).
// Entries at and beyond a group's rank are left unwritten: those kernels never read them.
int launch_transpose_job(const TransposeJob& t0, const int32_t* rank, int rpad, hipStream_t s) {
  if (t0.groups == 0) return TK_OK;
  TransposeJob t = t0;
  t.skip_dead = 1;
  const int64_t units = (int64_t)t.groups * rpad * ((t.bT ? t.out_features : 0) + t.in_features) / 64;  // 8 x 8 blocks
  const int64_t blocks = std::min<int64_t>(8192, std::max<int64_t>(1, units / 256));
  hipLaunchKernelGGL(k_transpose_job, dim3((unsigned)blocks), dim3(256), 0, s, t, rank, rpad);
  return check_launch();
}

// Shrink (with the slice sums) of n projections of one padded rank above 16 that read the same source.
int launch_shrink_multi(const PassArgs* a, int n, const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0 || n == 0) return TK_OK;
  PassJobs J{};
  for (int p = 0; p < n; ++p) J.p[p] = a[p];
  const int32_t* rows = seg.slot_table(a[0].map_rows);
  const bool quad = a[0].quad_steps > 0;
  const int items = (int)(ceil_div(L.max_tiles, quad ? 8 : 2) * a[0].kslices);
  const dim3 grid((unsigned)(ceil_div(items, 8) * 8 * n));
  if (quad) {  // the single-projection launch makes the same choice: same sums, same bits
    if (a[0].rpad <= 32)
      hipLaunchKernelGGL((k_shrink_quad_multi<2>), grid, dim3(256), 0, s, J, n, items, seg.tile_group, rows,
                         (int)L.max_tiles);
    else
      hipLaunchKernelGGL((k_shrink_quad_multi<4>), grid, dim3(256), 0, s, J, n, items, seg.tile_group, rows,
                         (int)L.max_tiles);
  } else if (a[0].rpad <= 32) {
    hipLaunchKernelGGL((k_shrink_pair_multi<2, 2>), grid, dim3(128), 0, s, J, n, items, seg.tile_group, rows,
                       (int)L.max_tiles);
  } else {
    hipLaunchKernelGGL((k_shrink_pair_multi<4, 4>), grid, dim3(256), 0, s, J, n, items, seg.tile_group, rows,
                       (int)L.max_tiles);
  }
  if (a[0].kslices > 1) {
    for (int p = 0; p < n; ++p) {
      bf16_t* hrow = (bf16_t*)a[p].hT + (int64_t)a[p].rpad * a[p].ldh;
      if (a[0].rpad <= 32)
        hipLaunchKernelGGL(k_shrink_finish<2>, dim3((unsigned)L.max_tiles), dim3(256), 0, s, a[p], hrow,
                           seg.tile_group, rows);
      else
        hipLaunchKernelGGL(k_shrink_finish<4>, dim3((unsigned)L.max_tiles), dim3(256), 0, s, a[p], hrow,
                           seg.tile_group, rows);
    }
  }
  return check_launch();
}

// Row contractions of n projections of one padded rank above 16 over the same source (see k_wgrad_coop_multi).
int launch_wgrad_coop_multi(const SharedWgradArgs& a0, const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0 || a0.nproj == 0) return TK_OK;
  SharedWgradArgs a = a0;
  for (int p = 0; p < a.nproj; ++p) a.w[p].tr = TransposeJob{};
  const int nx = a.w[0].width / 128;
  const int items = nx * (int)L.max_chunks;
  const dim3 grid((unsigned)(ceil_div(items, 8) * 8 * a.nproj));
  size_t dyn = (size_t)L.chunk_tiles * kTileRows * sizeof(int32_t);
  for (int p = 0; p < a.nproj; ++p)
    if (a.w[p].pair_chunks) dyn = 2 * (size_t)L.chunk_tiles * kTileRows * sizeof(int32_t);
  const int32_t* rows = seg.slot_table(a.w[0].map_rows);
  if (a.w[0].rpad <= 32)
    hipLaunchKernelGGL((k_wgrad_coop_multi<2, TK_COOP_STAGES>), grid, dim3(128), dyn, s, a, items, nx, seg.chunks, rows);
  else
    hipLaunchKernelGGL((k_wgrad_coop_multi<4, TK_COOP_STAGES>), grid, dim3(128), dyn, s, a, items, nx, seg.chunks, rows);
  return check_launch();
}

bool pass_mfma_supported(const PassArgs& a) {
  if (a.rpad > 64) return false;
  if (a.width_src % 64 != 0 || a.ld_src % 8 != 0 || !aligned16(a.src)) return false;
  if (a.dst && (a.width_dst % 128 != 0 || a.ld_dst % 8 != 0 || !aligned16(a.dst))) return false;
  if (a.ld_shrink % 8 != 0 || a.ld_expand % 8 != 0 || a.ldh % 8 != 0) return false;
  if (a.w_shrink_base && !aligned16(a.w_shrink_base)) return false;
  if (a.w_expand_base && !aligned16(a.w_expand_base)) return false;
  return true;
}

int launch_pass_mfma(const PassArgs& a, const SegView& seg, const SegLayout& L, int phases, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  if (a.rpad <= 16) launch_pass<1>(a, seg, L, phases, s);
  else if (a.rpad <= 32) launch_pass<2>(a, seg, L, phases, s);
  else launch_pass<4>(a, seg, L, phases, s);
  return check_launch();
}

bool wgrad_mfma_supported(const WgradArgs& a) {
  if (a.rpad > 64) return false;
  if (a.width % 128 != 0 || a.ld_src % 8 != 0 || a.ldh % 8 != 0 || !aligned16(a.src) || !aligned16(a.hT)) return false;
  return true;
}

int launch_wgrad_mfma(const WgradArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  if (a.rpad <= 16) launch_wgrad_pipe<1, TK_WGRAD_STAGES>(a, seg, L, s);
  else if (a.rpad <= 32) launch_wgrad_coop<2>(a, seg, L, s);
  else launch_wgrad_coop<4>(a, seg, L, s);
  return check_launch();
}

}  // namespace tk
