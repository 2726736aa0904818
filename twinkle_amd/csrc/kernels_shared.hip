// Projections that share their input (q / k / v, gate / up): the parts of the forward and backward
// passes that touch the shared tensors, done once for all of them.
//
//   forward   k_shrink_shared   x is read once and multiplied with every projection's A (the per-projection
//                               finish and expand kernels follow unchanged)
//   backward  k_expand_shared   dx += sum_p dh_p A_p in one read-modify-write of dx instead of one per projection
//             k_wgrad_shared    dA_p = dh_p^T x for every projection from one pass over x
//
// Each projection has padded rank 16 in these three, so projection p is simply block p of 16 rank indices of the
// single-projection kernels: same operand layouts, same order of every sum, hence the same h, dA and dB bit
// for bit; only dx differs (one rounding to bf16 instead of one per projection).
//
// At padded rank 32 and 64 a wave cannot hold several projections' operands at once.  There the single-projection
// shrink and row-contraction bodies are launched for all projections together, blocks that read the same piece of
// x next to each other on one XCD (k_shrink_pair_multi, k_wgrad_coop_multi in kernels_mfma.hip), and
//             k_expand_shared_hold   holds a wave's piece of dx in registers while the projections pass one after
//                                    the other: again one read-modify-write of dx.
#include "tk_mfma.h"

namespace tk {

namespace {

template <typename T>
__device__ inline T pick(const T (&v)[kMaxShared], int i) {  // v[i] without a register-indexed array
  T r = v[0];
#pragma unroll
  for (int j = 1; j < kMaxShared; ++j) r = i == j ? v[j] : r;
  return r;
}

// ---------------------------------------------------------------------------
// Shrink of P projections: work item = (two consecutive tiles, 512 source columns), one wave, exactly like
// k_shrink_pair<1, 1>; the wave keeps one accumulator block per projection and writes one slice of every
// projection's split-shrink buffer ([tile][slice][32][16] each), which that projection's k_shrink_finish
// turns into its h.
// ---------------------------------------------------------------------------
template <int P, int TT>
__device__ inline void shrink_tiles_shared(const SharedShrinkArgs& a, const int32_t* __restrict__ slot_rows,
                                           const int (&tiles)[TT], int g, int ks, float (*part)[16 * P + 1]) {
  constexpr int PF = P <= 2 ? 2 : 1;  // steps whose loads are issued together (what leaves three waves per SIMD)
  const int lane = threadIdx.x & 63, li = lane & 15, kb = lane >> 4;
  const bf16_t* src = (const bf16_t*)a.src;
  const bf16_t *xa[TT], *xb[TT];
#pragma unroll
  for (int u = 0; u < TT; ++u) {
    const int slot0 = tiles[u] * kTileRows;
    int ra = slot_rows[slot0 + li], rb = slot_rows[slot0 + 16 + li];
    ra = min(max(ra, 0), a.src_rows - 1);  // padding slots read a real row; their h is zeroed by the finish kernel
    rb = min(max(rb, 0), a.src_rows - 1);
    xa[u] = src + (int64_t)ra * a.ld_src + 16 * kb;
    xb[u] = src + (int64_t)rb * a.ld_src + 16 * kb;
  }
  const bf16_t* wp[P];
  bool wv[P];
  int r[P];
  bool any = false;
#pragma unroll
  for (int p = 0; p < P; ++p) {
    r[p] = min(a.rank[p][g], 16);
    any = any || r[p] > 0;
    wv[p] = li < r[p];
    wp[p] = (const bf16_t*)a.w[p][g] + (int64_t)(wv[p] ? li : 0) * a.ld_w[p] + 16 * kb;
  }
  f32x4 acc[TT][2][P];
#pragma unroll
  for (int u = 0; u < TT; ++u)
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int p = 0; p < P; ++p) acc[u][tt][p] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int nsteps = a.width_src >> 6;
  const int s_first = ks * kShrinkSteps;
#pragma unroll
  for (int b = 0; b < kShrinkSteps / PF; ++b) {
    uint4 x0[PF][TT][2], x1[PF][TT][2], w0[PF][P], w1[PF][P];
#pragma unroll
    for (int j = 0; j < PF; ++j) {
      const int s = s_first + b * PF + j;
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
      for (int p = 0; p < P; ++p) {
        w0[j][p] = (wv[p] && ok) ? ld16(wp[p] + c) : zero4();
        w1[j][p] = (wv[p] && ok) ? ld16(wp[p] + c + 8) : zero4();
      }
    }
#pragma unroll
    for (int j = 0; j < PF; ++j)
#pragma unroll
      for (int p = 0; p < P; ++p)
#pragma unroll
        for (int u = 0; u < TT; ++u)
#pragma unroll
          for (int tt = 0; tt < 2; ++tt) {
            acc[u][tt][p] = mfma16(x0[j][u][tt], w0[j][p], acc[u][tt][p]);
            acc[u][tt][p] = mfma16(x1[j][u][tt], w1[j][p], acc[u][tt][p]);
          }
  }
  if (!any) return;  // no projection's adapter is live on this layer (uniform over the block)
#pragma unroll
  for (int u = 0; u < TT; ++u) {
    __syncthreads();  // the previous tile's sums have been read
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int p = 0; p < P; ++p)
#pragma unroll
        for (int v = 0; v < 4; ++v) part[16 * tt + 4 * kb + v][16 * p + li] = acc[u][tt][p][v];
    __syncthreads();
#pragma unroll
    for (int p = 0; p < P; ++p) {
      if (r[p] <= 0) continue;
      float* mine = a.hpart[p] + ((int64_t)tiles[u] * a.kslices + ks) * (kTileRows * 16);
      for (int idx = lane; idx < kTileRows * 16; idx += 64) mine[idx] = part[idx >> 4][16 * p + (idx & 15)];
    }
  }
}

template <int P>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(P <= 3 ? 3 : 2))) void k_shrink_shared(SharedShrinkArgs a, const int32_t* __restrict__ tile_group,
                                                      const int32_t* __restrict__ slot_rows, int max_tiles) {
  __shared__ float part[kTileRows][16 * P + 1];
  const int block = xcd_contiguous(blockIdx.x, gridDim.x);
  const int pair = block / a.kslices, ks = block - pair * a.kslices;
  const int t0 = 2 * pair, t1 = t0 + 1;
  if (t0 >= max_tiles) return;
  const int g0 = checked_group(tile_group[t0], a.tb);
  const int g1 = t1 < max_tiles ? checked_group(tile_group[t1], a.tb) : -1;
  if (g0 >= 0 && g1 == g0) {
    const int tiles[2] = {t0, t1};
    shrink_tiles_shared<P, 2>(a, slot_rows, tiles, g0, ks, part);
    return;
  }
  if (g0 >= 0) {
    const int tiles[1] = {t0};
    shrink_tiles_shared<P, 1>(a, slot_rows, tiles, g0, ks, part);
  }
  if (g1 >= 0) {
    const int tiles[1] = {t1};
    shrink_tiles_shared<P, 1>(a, slot_rows, tiles, g1, ks, part);
  }
}

// ---------------------------------------------------------------------------
// dx[row] += sum_p dh_p[row] A_p: the flat expand kernel (one wave = one tile x 128 columns) with the
// contraction running over the P projections' blocks of 16 rank indices; lane group kb reads block
// 2 ks + kb / 2 of h (slot-major, [slots][16] per projection) and of the transposed weight copies
// ([G][K][16] per projection, rows permuted inside every 128 as TransposeJob::swizzle_a describes).
// ---------------------------------------------------------------------------
template <int P>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3))) void k_expand_shared(SharedExpandArgs a, const int32_t* __restrict__ tile_group,
                                                       const int32_t* __restrict__ slot_rows, int num_items) {
  constexpr int NKS = (16 * P + 31) / 32;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const int ngroups = a.width_dst >> 7;
  const int item = xcd_contiguous(blockIdx.x, gridDim.x) * 4 + wave;
  if (item >= num_items) return;
  const int tile_id = item / ngroups;
  const int c0 = (item - tile_id * ngroups) << 7;
  const int slot0 = tile_id * kTileRows;
  const int g_raw = checked_group(tile_group[tile_id], a.tb);
  const int4 r0 = *reinterpret_cast<const int4*>(slot_rows + slot0 + 4 * kb);
  const int4 r1 = *reinterpret_cast<const int4*>(slot_rows + slot0 + 16 + 4 * kb);
  const int off = 8 * (kb & 1);  // first rank index of this lane inside its block
  uint4 hop[2][NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    const int blk = 2 * ks + (kb >> 1);
    const bf16_t* hp = (const bf16_t*)pick(a.hrow, blk);
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
      hop[tt][ks] = blk < P ? ld16(hp + (int64_t)(slot0 + 16 * tt + li) * 16 + off) : zero4();
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
  int rblk[NKS];
  bool any = false;
#pragma unroll
  for (int p = 0; p < P; ++p) any = any || (g_raw >= 0 && a.rank[p][g] > 0);
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    const int blk = 2 * ks + (kb >> 1);
    rblk[ks] = (blk < P && g_raw >= 0) ? min(pick(a.rank, blk)[g], 16) : 0;
  }
  uint4 y[2][4];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int v = 0; v < 4; ++v) y[tt][v] = rok[tt][v] ? ld16_nt(yp[tt][v]) : zero4();
  uint4 bq[8][NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    const int blk = 2 * ks + (kb >> 1);
    // rows permuted inside every 128: the row of column c0 + 8 li + q lies at c0 + 16 q + li
    const bf16_t* wt = (const bf16_t*)pick(a.aT, blk) + ((int64_t)g * a.width_dst + c0 + li) * 16 + off;
#pragma unroll
    for (int q = 0; q < 8; ++q)
      bq[q][ks] = off < rblk[ks] ? keep_first(ld16(wt + (int64_t)q * 256), rblk[ks] - off) : zero4();
  }
  if (!any) return;  // unused tile, or no projection live on this layer (uniform over the wave)
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks)  // a projection without this adapter has no dh: never multiply what is there
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) hop[tt][ks] = rblk[ks] > 0 ? hop[tt][ks] : zero4();
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

// ---------------------------------------------------------------------------
// dA_p[n][c] = sum over the rows of dh_p[n][slot] x[row(slot)][c] for all projections from one pass over x:
// k_wgrad_pipe's pipeline and operand layouts with one accumulator block per projection; every block
// leaves through the same staging buffer into its own projection's partial buffer or gradient.
// ---------------------------------------------------------------------------
template <int P>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(P <= 3 ? 2 : 1))) void k_wgrad_shared(
    SharedWgradArgs a, const ChunkInfo* __restrict__ chunks, const int32_t* __restrict__ slot_rows) {
  constexpr int OS = kWgradStageStride;
  constexpr int STAGES = 2;  // tiles in registers: what fits next to P accumulator blocks at two waves per SIMD
  __shared__ __attribute__((aligned(16))) float lds[16 * OS];
  extern __shared__ __attribute__((aligned(16))) int32_t rows_s[];  // the chunk's row indices
  const int lane = threadIdx.x & 63, li = lane & 15, kb = lane >> 4;
  const int c0 = blockIdx.x * 128;
  const ChunkInfo ci = checked_chunk(chunks[blockIdx.y], a.w[0].tb);
  const int g = ci.group;
  if (g < 0) return;
  int r[P];
  bool any = false;
#pragma unroll
  for (int p = 0; p < P; ++p) {
    r[p] = min(a.w[p].rank[g], 16);
    any = any || r[p] > 0;
  }
  if (!any) return;
  const WgradArgs& a0 = a.w[0];
  const int nt = ci.ntiles;
  // the row indices go through LDS: reading them there does not wait for the tile loads in flight
  for (int i = lane; i < nt * kTileRows; i += 64) rows_s[i] = slot_rows[ci.tile0 * kTileRows + i];
  const bf16_t* src = (const bf16_t*)a0.src + c0 + 8 * li;
  const bf16_t* hT[P];
#pragma unroll
  for (int p = 0; p < P; ++p)
    hT[p] = (const bf16_t*)a.w[p].hT + (int64_t)li * a.w[p].ldh + (int64_t)ci.tile0 * kTileRows + 8 * kb;
  f32x4 acc[8][P];
#pragma unroll
  for (int q = 0; q < 8; ++q)
#pragma unroll
    for (int p = 0; p < P; ++p) acc[q][p] = f32x4{0.f, 0.f, 0.f, 0.f};
  __syncthreads();

  struct Tile {
    uint4 x[8];
    uint4 h[P];
    uint32_t live;
  };
  // loads are unconditional (tiles past the end re-read the last one, padding slots read row 0); what must
  // not count is zeroed when it is consumed
  auto issue = [&](int t, Tile& T) {
    const int tc = min(t, nt - 1);
    const int4 ra = *reinterpret_cast<const int4*>(rows_s + tc * kTileRows + 8 * kb);
    const int4 rb = *reinterpret_cast<const int4*>(rows_s + tc * kTileRows + 8 * kb + 4);
    const int rows[8] = {ra.x, ra.y, ra.z, ra.w, rb.x, rb.y, rb.z, rb.w};
    T.live = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int row = checked_row(rows[q], a0.tb);
      T.x[q] = ld16(src + (int64_t)max(row, 0) * a0.ld_src);
      T.live |= (t < nt && row >= 0) ? (1u << q) : 0u;
    }
#pragma unroll
    for (int p = 0; p < P; ++p) T.h[p] = ld16(hT[p] + tc * kTileRows);
  };
  auto consume = [&](const Tile& T) {
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
      for (int p = 0; p < P; ++p) acc[q][p] = mfma16(tr, T.h[p], acc[q][p]);
    }
  };
  if constexpr (STAGES == 3) {
    Tile A, B, C;
    issue(0, A);
    issue(1, B);
    int t = 0;
    for (; t + 4 < nt; t += 3) {  // every tile touched in here exists
      issue(t + 2, C);
      consume(A);
      issue(t + 3, A);
      consume(B);
      issue(t + 4, B);
      consume(C);
    }
    issue(t + 2, C);
    consume(A);
    consume(B);
    consume(C);
    if (t + 3 < nt) {
      issue(t + 3, A);
      consume(A);
    }
  } else {
    Tile A, B;
    issue(0, A);
    int t = 0;
    for (; t + 2 < nt; t += 2) {
      issue(t + 1, B);
      consume(A);
      issue(t + 2, A);
      consume(B);
    }
    issue(t + 1, B);  // one or two tiles are left
    consume(A);
    consume(B);       // all zeros when tile t + 1 does not exist
  }
#pragma unroll
  for (int p = 0; p < P; ++p) {
    if (r[p] <= 0) continue;
    f32x4 one[8][1];
#pragma unroll
    for (int q = 0; q < 8; ++q) one[q][0] = acc[q][p];
    wgrad_store<1>(one, lds, a.w[p], ci, g, r[p], c0, lane);
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");  // the staging buffer is read before the next block overwrites it
  }
}

// ---------------------------------------------------------------------------
// dx[row] += sum_p dh_p[row] A_p for projections of padded rank 32 or 64, with the weights held across tiles (what
// k_expand_multi does for one projection): one wave = two consecutive tiles x 128 columns.  Weights come from the
// transposed copies [G][K][rpad] of every projection (not permuted).  Its piece of dx stays in registers as bf16 (64 registers) while the
// projections pass one after the other: per projection the wave loads the 128 x rank block of A^T once for both
// tiles (as long as they belong to one group), multiplies each tile's dh_p with it and adds the product onto the
// held rows, rounding to bf16 after every projection exactly as one k_expand_multi launch per projection would: dx
// has the bits of the separate calls, with one read and one write of dx instead of one per projection.  (A form with
// one tile per wave and fp32 sums over the projections fetched every weight block once per tile; the traffic
// between L2 and the CUs bounds these kernels above rank 16, and it took 155 us against 123 us for this one at
// q / k / v of rank 64, 16384 rows; three k_expand_multi launches: 135 us.)
// Items are numbered by sets of four tiles (the segment table's set order when rows are gathered and the keys were
// interleaved, contiguous runs per XCD otherwise, as in k_expand_multi), each set as two halves.
// ---------------------------------------------------------------------------
template <int NB>
__global__ __launch_bounds__(256) void k_expand_shared_hold(SharedExpandArgs a, const int32_t* __restrict__ tile_group,
                                                            const int32_t* __restrict__ slot_rows,
                                                            const int32_t* __restrict__ set_walk,
                                                            const SegHeader* __restrict__ header,
                                                            const uint8_t* __restrict__ round_moved, int sort_blocks,
                                                            int max_tiles) {
  constexpr int RP = 16 * NB, NKS = RP / 32, TPI = 2;
  // The four waves of a block update the same two tiles (128 columns each), so they multiply with the same dh
  // operands: these are fetched once per block into LDS (the two tiles' 64 slots x RP of every projection: one
  // contiguous run of hrow each) instead of once per wave.  Row stride RP + 8 elements: operand reads without bank
  // conflicts.
  constexpr int HS = RP + 8;
  __shared__ __attribute__((aligned(16))) bf16_t dh_s[kMaxShared][TPI * kTileRows * HS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const int ngroups = a.width_dst >> 7;
  const int nbt = (ngroups + 3) >> 2;  // blocks per pair of tiles: column block fastest
  const int per_set = nbt * (kSetTiles / TPI);
  int swept_set = 0;
  bool sweep = false;
  if (set_walk != nullptr) {
    swept_set = set_walk[blockIdx.x / per_set];
    uint2 moved = make_uint2(0u, 0u);
    if (lane < sort_blocks) moved = reinterpret_cast<const uint2*>(round_moved)[lane];
    sweep = header->identity_order == 0 && __ballot((moved.x | moved.y) != 0u) != 0ull;
  }
  const int block = sweep ? (int)blockIdx.x : xcd_contiguous(blockIdx.x, gridDim.x);
  const int in_set = block % per_set, set = block / per_set;
  const int cb = in_set % nbt, half = in_set / nbt;
  const int tile0 = (sweep ? swept_set : set) * kSetTiles + half * TPI;
  const int cg = cb * 4 + wave;
  if ((unsigned)tile0 >= (unsigned)max_tiles) return;  // (uniform over the block, like the next return)
  const int nt = min(TPI, max_tiles - tile0);
  int gt[TPI];
#pragma unroll
  for (int t = 0; t < TPI; ++t) gt[t] = t < nt ? checked_group(tile_group[tile0 + t], a.tb) : -1;
  if (gt[0] < 0 && gt[1] < 0) return;
  {
    // 16-byte pieces of the nt tiles' dh rows, all projections' requested together
    constexpr int PPR = RP / 8;                       // pieces per row
    constexpr int PIECES = TPI * kTileRows * PPR;     // per projection
    constexpr int PER = (PIECES + 255) / 256;
    uint4 v[kMaxShared][PER];
#pragma unroll
    for (int p = 0; p < kMaxShared; ++p) {
      const bf16_t* hp = (const bf16_t*)pick(a.hrow, p) + (int64_t)tile0 * kTileRows * RP;
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int e = tid + 256 * i;
        v[p][i] = (p < a.nproj && e < nt * kTileRows * PPR) ? ld16(hp + 8 * e) : zero4();
      }
    }
#pragma unroll
    for (int p = 0; p < kMaxShared; ++p)
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int e = tid + 256 * i;
        if (e < PIECES) st16(&dh_s[p][(e / PPR) * HS + 8 * (e % PPR)], v[p][i]);
      }
  }
  __syncthreads();
  if (cg >= ngroups) return;  // a column group past the width (after the block's only barrier)
  const int c0 = cg << 7;
  bf16_t* dst = (bf16_t*)a.dst + c0 + 8 * li;
  // the rows this lane updates (slots 16 tt + 4 kb + v of each tile) and their dx
  int rows[TPI][2][4];
  uint4 y[TPI][2][4];
#pragma unroll
  for (int t = 0; t < TPI; ++t) {
    const bool tok = gt[t] >= 0;  // wave-uniform
    const unsigned row_limit = tok ? (unsigned)a.tb.rows : 0u;
    const int slot0 = (tile0 + (t < nt ? t : 0)) * kTileRows;
    const int4 r0 = *reinterpret_cast<const int4*>(slot_rows + slot0 + 4 * kb);
    const int4 r1 = *reinterpret_cast<const int4*>(slot_rows + slot0 + 16 + 4 * kb);
    const int rr[2][4] = {{r0.x, r0.y, r0.z, r0.w}, {r1.x, r1.y, r1.z, r1.w}};
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        rows[t][tt][v] = (unsigned)rr[tt][v] < row_limit ? rr[tt][v] : -1;
        y[t][tt][v] = rows[t][tt][v] >= 0 ? ld16_nt(dst + (int64_t)rows[t][tt][v] * a.ld_dst) : zero4();
      }
  }
  bool touched[TPI] = {false, false};
  for (int p = 0; p < a.nproj; ++p) {
    const int32_t* rank = pick(a.rank, p);
    const bf16_t* hp = dh_s[p];
    const bf16_t* wT = (const bf16_t*)pick(a.aT, p);
    int held = -1, r = 0;
    uint4 bq[8][NKS];
#pragma unroll
    for (int t = 0; t < TPI; ++t) {
      const int g = gt[t];
      if (g < 0) continue;  // (uniform over the wave, like every branch of this loop)
      uint4 hop[2][NKS];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
          hop[tt][ks] = ld16(hp + (t * kTileRows + 16 * tt + li) * HS + 32 * ks + 8 * kb);
      if (g != held) {
        held = g;
        r = min(rank[g], RP);
        const bf16_t* wt = wT + ((int64_t)g * a.width_dst + c0 + 8 * li) * RP;
#pragma unroll
        for (int q = 0; q < 8; ++q)
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            const int n0 = 32 * ks + 8 * kb;
            bq[q][ks] = n0 < r ? keep_first(ld16(wt + (int64_t)q * RP + n0), r - n0) : zero4();
          }
      }
      if (r <= 0) continue;  // the group's adapter is not live in this projection
      touched[t] = true;
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
          const uint4 yy = y[t][tt][v];
          uint4 o;
          o.x = pack_bf16(bf16_lo(yy.x) + d[0][v], bf16_hi(yy.x) + d[1][v]);
          o.y = pack_bf16(bf16_lo(yy.y) + d[2][v], bf16_hi(yy.y) + d[3][v]);
          o.z = pack_bf16(bf16_lo(yy.z) + d[4][v], bf16_hi(yy.z) + d[5][v]);
          o.w = pack_bf16(bf16_lo(yy.w) + d[6][v], bf16_hi(yy.w) + d[7][v]);
          y[t][tt][v] = o;
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < TPI; ++t) {
    if (!touched[t]) continue;
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int v = 0; v < 4; ++v)
        if (rows[t][tt][v] >= 0) st16_nt(dst + (int64_t)rows[t][tt][v] * a.ld_dst, y[t][tt][v]);
  }
}

}  // namespace

int launch_expand_shared_wide(const SharedExpandArgs& a, int rpad, const SegView& seg, const SegLayout& L,
                              hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  const int32_t* rows = seg.slot_table(a.map_rows);
  const int64_t nbt = ceil_div((int64_t)(a.width_dst >> 7), 4);
  const dim3 grid((unsigned)(ceil_div(L.max_tiles, kSetTiles) * (kSetTiles / 2) * nbt));
  const int sb = (int)std::min<int64_t>(L.sort_blocks, 64);
  if (rpad <= 32)
    hipLaunchKernelGGL(k_expand_shared_hold<2>, grid, dim3(256), 0, s, a, seg.tile_group, rows,
                       seg.set_walk(a.map_rows), seg.header, seg.round_moved, sb, (int)L.max_tiles);
  else
    hipLaunchKernelGGL(k_expand_shared_hold<4>, grid, dim3(256), 0, s, a, seg.tile_group, rows,
                       seg.set_walk(a.map_rows), seg.header, seg.round_moved, sb, (int)L.max_tiles);
  return check_launch();
}

int launch_shrink_shared(const SharedShrinkArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  const dim3 grid((unsigned)(ceil_div(L.max_tiles, 2) * a.kslices));
  const int32_t* rows = seg.slot_table(a.map_rows);
  if (a.nproj == 2)
    hipLaunchKernelGGL(k_shrink_shared<2>, grid, dim3(64), 0, s, a, seg.tile_group, rows, (int)L.max_tiles);
  else if (a.nproj == 3)
    hipLaunchKernelGGL(k_shrink_shared<3>, grid, dim3(64), 0, s, a, seg.tile_group, rows, (int)L.max_tiles);
  else
    hipLaunchKernelGGL(k_shrink_shared<4>, grid, dim3(64), 0, s, a, seg.tile_group, rows, (int)L.max_tiles);
  return check_launch();
}

int launch_expand_shared(const SharedExpandArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  const int64_t items = L.max_tiles * (a.width_dst >> 7);
  const dim3 grid((unsigned)ceil_div(items, 4));
  const int32_t* rows = seg.slot_table(a.map_rows);
  if (a.nproj == 2)
    hipLaunchKernelGGL(k_expand_shared<2>, grid, dim3(256), 0, s, a, seg.tile_group, rows, (int)items);
  else if (a.nproj == 3)
    hipLaunchKernelGGL(k_expand_shared<3>, grid, dim3(256), 0, s, a, seg.tile_group, rows, (int)items);
  else
    hipLaunchKernelGGL(k_expand_shared<4>, grid, dim3(256), 0, s, a, seg.tile_group, rows, (int)items);
  return check_launch();
}

int launch_wgrad_shared(const SharedWgradArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  const dim3 grid((unsigned)(a.w[0].width / 128), (unsigned)L.max_chunks);
  const int32_t* rows = seg.slot_table(a.w[0].map_rows);
  const size_t dyn = (size_t)L.chunk_tiles * kTileRows * sizeof(int32_t);  // a chunk's row indices
  if (a.nproj == 2)
    hipLaunchKernelGGL(k_wgrad_shared<2>, grid, dim3(64), dyn, s, a, seg.chunks, rows);
  else if (a.nproj == 3)
    hipLaunchKernelGGL(k_wgrad_shared<3>, grid, dim3(64), dyn, s, a, seg.chunks, rows);
  else
    hipLaunchKernelGGL(k_wgrad_shared<4>, grid, dim3(64), dyn, s, a, seg.chunks, rows);
  return check_launch();
}


}  // namespace tk
