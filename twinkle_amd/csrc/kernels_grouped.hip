// Grouped base GEMM of packed experts with the LoRA term in its epilogue (gfx950, bf16 MFMA).
//
//   y[row(slot)][n] = sum_k x[row(slot)][k] * W_e[n][k]  (+ sum_r h[slot][r] * B_g[n][r])
//
// for every slot of the segment table, e = g / groups_per_weight the weight (expert) of the slot's group g.
// One launch serves all experts: the reference loops over the experts on the host and synchronises for each
// chunk boundary.  The LoRA term enters as extra contraction steps on the accumulators, so y is written once
// instead of written by the GEMM and then read, updated and written again by the expand kernel.
//
//   k_grouped_plan      one small block: the list of row blocks (up to 4 or 8 consecutive tiles of one expert, an
//                       expert's tiles cut into blocks of equal length)
//   k_grouped_gemm_dl   out_features a multiple of 256 and operands under 4 GB: block tile 256 x 256 x 64, eight
//                       waves, the operand tiles loaded from global memory straight into LDS (both weight layouts,
//                       with and without the LoRA term); described where it is defined
//   k_grouped_gemm      the rest: operands through registers into LDS; 8 waves on 256 x 256 tiles or 4 waves on
//                       128 x 128 (row stride 144 B in LDS: conflict-free 16-byte operand reads, a wave owns
//                       64 x 64 as 4 x 4 MFMA 16x16x32 tiles)
//
// A block takes one row block and a run of column blocks of the output: the row block's x stays in L2 across the
// column blocks, and the row blocks of one expert, which reach an XCD together, stream that expert's weights through
// the XCD's L2 side by side.  The weight fragment is the MFMA A operand and the x fragment the B operand, so a lane
// ends up with four consecutive output columns of one row.
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "tk_mfma.h"

namespace tk {

namespace {

constexpr int kGBK = 64, kGLS = kGBK + 8;
#ifndef TK_GROUPED_ITEMS
#define TK_GROUPED_ITEMS 6144
#endif
#ifndef TK_GROUPED_BIG
#define TK_GROUPED_BIG 1
#endif
#ifndef TK_GROUPED_DL
#define TK_GROUPED_DL 1  // 8 waves, 256 x 256 tiles: operand tiles go from global memory straight into LDS
#endif
constexpr int kGroupedItems = TK_GROUPED_ITEMS;  // work items aimed at per launch

__global__ __launch_bounds__(256) void k_grouped_plan(const int32_t* __restrict__ tile_first, int experts, int nt,
                                                      GroupedPlanEntry* __restrict__ plan,
                                                      int32_t* __restrict__ nblocks, int max_entries, int ptiles,
                                                      int max_tiles) {
  __shared__ int32_t sums[256];
  const int tid = threadIdx.x;
  const int per = (experts + 255) / 256;
  const int e0 = min(experts, tid * per), e1 = min(experts, e0 + per);
  int cnt = 0;
  // (tile numbers come from the caller's segment table: kept inside [0, max_tiles] and ascending before they index)
  auto first_tile = [&](int g) { return min(max(tile_first[g], 0), max_tiles); };
  for (int e = e0; e < e1; ++e) cnt += (max(first_tile((e + 1) * nt) - first_tile(e * nt), 0) + ptiles - 1) / ptiles;
  sums[tid] = cnt;
  __syncthreads();
  for (int off = 1; off < 256; off <<= 1) {
    const int v = tid >= off ? sums[tid - off] : 0;
    __syncthreads();
    sums[tid] += v;
    __syncthreads();
  }
  int at = sums[tid] - cnt;
  for (int e = e0; e < e1; ++e) {
    const int t0 = first_tile(e * nt), t1 = max(first_tile((e + 1) * nt), t0);
    // the expert's tiles in `count` row blocks of (almost) equal length: blocks of equal work stay in step, and
    // blocks in step find each other's weight and x tiles in the XCD's L2 (measured at config 4, 18 tiles per expert:
    // as 8 + 8 + 2 the short block runs ahead and L2 fetches 1.6 x the compulsory bytes, as 6 + 6 + 6 it fetches
    // 1.2 x)
    const int first = at, count = (t1 - t0 + ptiles - 1) / ptiles;
    const int per = count > 0 ? (t1 - t0 + count - 1) / count : ptiles;
    for (int t = t0; t < t1; t += per, ++at)
      if (at < max_entries) plan[at] = GroupedPlanEntry{t, min(per, t1 - t), e, first, count, 0};
  }
  if (tid == 255) *nblocks = min(sums[255], max_entries);
}

// NKS: MFMA steps of the LoRA term (0: none; 1: padded rank 16 or 32; 2: padded rank 64)
// BIG: 0: 4 waves (2 x 2), wave tile 64 x 64, block tile 128 x 128, two blocks per CU, loads two steps ahead;
//      1: 8 waves (2 x 4), wave tile 128 x 64, block tile 256 x 256, one block per CU: half the operand bytes per
//         FLOP out of L2 and three LDS reads per eight MFMAs instead of four; a wave whose rows are dead (the tail
//         of an expert) skips its MFMAs, so a half-empty block takes about half the time
// TR:  0: weight rows are output features (y = x W^T, the contraction runs along the weight's rows in memory);
//      1: weight rows are input features (y = x W: the backward of TR = 0 on the same memory).  The lower half of
//         the block then loads the weight tile as 8 x 8 blocks, transposes them in registers and writes them to LDS
//         with the 16-byte chunks of a row XOR-swizzled by the row's block number (conflict-free on both sides);
//         the upper half loads the x tile.
template <int NKS, int BIG, int TR>
__global__ __launch_bounds__(BIG ? 512 : 256) __attribute__((amdgpu_waves_per_eu(2))) void k_grouped_gemm(
    GroupedArgs a, const GroupedPlanEntry* __restrict__ plan, const int32_t* __restrict__ nblocks,
    const int32_t* __restrict__ tile_group, const int32_t* __restrict__ slot_rows, int nsplit, int cpi) {
  constexpr int THREADS = BIG ? 512 : 256, WN = BIG ? 4 : 2, RB = BIG ? 8 : 4, CB = 4;
  constexpr int BM = 2 * 16 * RB, BN = WN * 16 * CB;  // 128 x 128 or 256 x 256
  constexpr int LROWS = THREADS / 8;                   // rows moved per pass of the block's loads
  constexpr int XP = BM / LROWS, WP = BN / LROWS;      // passes: 4 and 4
  constexpr int SETS = (BIG || TR) ? 1 : 2;            // register sets of loads in flight
  __shared__ __attribute__((aligned(16))) bf16_t As[2][BM * kGLS];  // x rows
  __shared__ __attribute__((aligned(16))) bf16_t Bs[2][BN * kGLS];  // weight rows
  // work item = (row block, run of cpi column blocks); the items of one expert are neighbours and reach one XCD
  // together
  const int blocks = *nblocks * nsplit;
  if ((int)blockIdx.x >= blocks) return;
  const int item = xcd_contiguous(blockIdx.x, blocks);
  // within an expert: column run major, row block minor, so that the blocks that read the same weight rows start
  // side by side (the expert's entries are contiguous: any of them names the range)
  const GroupedPlanEntry any = plan[item / nsplit];
  const int local = item - any.first * nsplit;
  const GroupedPlanEntry pe = plan[any.first + local % any.count];
  const int nb_first = (local / any.count) * cpi, nb_last = min(nb_first + cpi, a.N / BN);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const int wm = wave / WN, wn = wave % WN;
  const int slot0 = pe.tile0 * kTileRows, live = pe.ntiles * kTileRows;
  const int live_w = min(max(live - 16 * RB * wm, 0), 16 * RB);  // live rows of this wave's strip (uniform)

  // global -> LDS (TR = 0): thread t moves 16 bytes of rows (t >> 3) + LROWS i at column chunk t & 7, of x and of
  // the weights alike.  (TR = 1): the upper half of the threads does that for x alone (XR rows per pass, 8 passes),
  // the lower half owns one 8 x 8 block of the weight tile each.
  constexpr int XR = TR ? THREADS / 16 : LROWS, XN = TR ? 8 : XP;
  const bool w_thread = TR && tid < THREADS / 2;           // uniform over a wave
  const int xt = TR ? (tid & (THREADS / 2 - 1)) : tid;
  const int lrow = xt >> 3, lchunk = (xt & 7) * 8;
  const bf16_t* xp[XN];
#pragma unroll
  for (int i = 0; i < XN; ++i) {
    const int r = lrow + XR * i;
    int row = r < live ? slot_rows[slot0 + r] : -1;  // padding and dead rows read row 0 and are never stored
    row = min(max(row, 0), a.src_rows - 1);
    xp[i] = a.x + (int64_t)row * a.ldx + lchunk;
  }
  const int cblk = tid / (BN / 8), jblk = tid % (BN / 8);  // TR: this thread's block of the weight tile
  // rows this lane stores: slots 16 RB wm + 16 rb + li
  int out_row[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int r = 16 * RB * wm + 16 * rb + li;
    out_row[rb] = r < live ? checked_row(slot_rows[slot0 + r], a.tb) : -1;
  }
  const bf16_t* wbase = a.w + (int64_t)pe.expert * a.w_stride;
  const int nk = a.K / kGBK;
  const int ldsw = lrow * kGLS + lchunk;  // + LROWS i rows

  for (int nb = nb_first; nb < nb_last; ++nb) {
    const bf16_t* wp[TR ? 1 : WP];
    if constexpr (TR) {
      wp[0] = wbase + (int64_t)(8 * cblk) * a.ldw + nb * BN + 8 * jblk;
    } else {
#pragma unroll
      for (int i = 0; i < WP; ++i) wp[i] = wbase + (int64_t)(nb * BN + lrow + LROWS * i) * a.ldw + lchunk;
    }
    f32x4 acc[RB][CB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) acc[rb][cb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // The loads of step ks + SETS are issued before step ks is computed and wait in registers across the barrier
    // (which orders LDS traffic only).
    uint4 gx[SETS][TR ? 8 : XP], gw[SETS][TR ? 1 : WP];  // TR: gx holds a thread's eight pieces of either tile
    auto fetch = [&](int ks, auto set) {
      const int k0 = ks * kGBK;
      if constexpr (TR) {
        if (w_thread) {
          const bf16_t* p = wp[0] + (int64_t)k0 * a.ldw;
#pragma unroll
          for (int i = 0; i < 8; ++i) gx[set][i] = ld16(p + (int64_t)i * a.ldw);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) gx[set][i] = ld16(xp[i] + k0);
        }
      } else {
#pragma unroll
        for (int i = 0; i < XP; ++i) gx[set][i] = ld16(xp[i] + k0);
#pragma unroll
        for (int i = 0; i < WP; ++i) gw[set][i] = ld16(wp[i] + k0);
      }
    };
    auto stash = [&](int buf, auto set) {
      if constexpr (TR) {
        if (w_thread) {
          // 8 x 8 transpose inside the thread: piece q becomes column q of the block, the eight contraction indices
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const int d = q >> 1;
            const uint32_t sel = (q & 1) ? 0x07060302u : 0x05040100u;
            uint32_t e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              const uint32_t wsrc[4] = {gx[set][i].x, gx[set][i].y, gx[set][i].z, gx[set][i].w};
              e[i] = wsrc[d];
            }
            uint4 tr;
            tr.x = __builtin_amdgcn_perm(e[1], e[0], sel);
            tr.y = __builtin_amdgcn_perm(e[3], e[2], sel);
            tr.z = __builtin_amdgcn_perm(e[5], e[4], sel);
            tr.w = __builtin_amdgcn_perm(e[7], e[6], sel);
            st16(&Bs[buf][(8 * jblk + q) * kGLS + 8 * (cblk ^ (jblk & 7))], tr);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) st16(&As[buf][ldsw + XR * i * kGLS], gx[set][i]);
        }
      } else {
#pragma unroll
        for (int i = 0; i < XP; ++i) st16(&As[buf][ldsw + LROWS * i * kGLS], gx[set][i]);
#pragma unroll
        for (int i = 0; i < WP; ++i) st16(&Bs[buf][ldsw + LROWS * i * kGLS], gw[set][i]);
      }
    };
    auto step = [&](int ks, auto parity) {  // parity = ks & 1 as a compile-time constant
      constexpr int cur = decltype(parity)::value;
      if (ks + SETS < nk) fetch(ks + SETS, std::integral_constant<int, SETS == 2 ? cur : 0>{});
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        uint4 fw[CB];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
          const int j = 16 * CB * wn + 16 * cb + li;
          const int chunk = TR ? ((4 * s + kb) ^ ((j >> 3) & 7)) : 4 * s + kb;
          fw[cb] = ld16(&Bs[cur][j * kGLS + 8 * chunk]);
        }
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          if (16 * rb >= live_w) break;
          const uint4 fx = ld16(&As[cur][(16 * RB * wm + 16 * rb + li) * kGLS + 32 * s + 8 * kb]);
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) acc[rb][cb] = mfma16(fw[cb], fx, acc[rb][cb]);
        }
      }
      if (ks + 1 < nk) stash(cur ^ 1, std::integral_constant<int, SETS == 2 ? (cur ^ 1) : 0>{});
      lds_barrier();
    };
    fetch(0, std::integral_constant<int, 0>{});
    if (SETS == 2 && nk > 1) fetch(1, std::integral_constant<int, SETS - 1>{});
    stash(0, std::integral_constant<int, 0>{});
    lds_barrier();
    for (int ks = 0; ks < nk; ks += 2) {
      step(ks, std::integral_constant<int, 0>{});
      if (ks + 1 < nk) step(ks + 1, std::integral_constant<int, 1>{});
    }

    if constexpr (NKS > 0) {
      // LoRA term: h[slot][0 .. rpad) against B_g[n][0 .. rank), per 32-row tile (a tile has one group)
#pragma unroll
      for (int tl = 0; tl < RB / 2; ++tl) {
        const int tile_in_block = (RB / 2) * wm + tl;
        if (tile_in_block >= pe.ntiles) break;
        const int g = checked_group(tile_group[pe.tile0 + tile_in_block], a.tb);
        const int r = g >= 0 ? min(a.rank[g], a.rpad) : 0;
        if (r <= 0) continue;
        const bf16_t* Bg = (const bf16_t*)a.lora_B[g];
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
          const int n0 = 32 * s + 8 * kb;  // first rank index of this lane's operand piece
          if (32 * s >= r) break;          // uniform over the wave
          uint4 fh[2], fb[CB];
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const int slot = slot0 + 32 * tile_in_block + 16 * q + li;
            fh[q] = n0 < a.rpad ? ld16(a.hrow + (int64_t)slot * a.rpad + n0) : zero4();
          }
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) {
            const int n = nb * BN + 16 * CB * wn + 16 * cb + li;
            fb[cb] = n0 < r ? keep_first(ld16(Bg + (int64_t)n * a.ldb + n0), r - n0) : zero4();
          }
#pragma unroll
          for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) acc[2 * tl + q][cb] = mfma16(fb[cb], fh[q], acc[2 * tl + q][cb]);
        }
      }
    }

    // lane holds y[slot 16 RB wm + 16 rb + li][nb BN + 16 CB wn + 16 cb + 4 kb + v], v = 0..3: 8-byte stores
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      if (out_row[rb] < 0) continue;
      bf16_t* yp = a.y + (int64_t)out_row[rb] * a.ldy + nb * BN + 16 * CB * wn + 4 * kb;
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        const f32x4 v = acc[rb][cb];
        *reinterpret_cast<uint2*>(yp + 16 * cb) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The same product with the operand tiles going from global memory straight into LDS (global_load_lds, 16 bytes per
// lane): no staging registers and no LDS stores, so the wave has room for all operand fragments of a 32-deep half
// step (12 x 16 bytes per lane) and reads them ahead of the MFMAs that use them.  Block tile 256 x 256 x 64, eight
// waves (2 x 4), wave tile 128 x 64, two stages of 64 KB.
//
// Stage layout: x rows and weight rows alike, row r of the tile at byte 128 r, its 16-byte chunk c at position
// c ^ (r & 7).  A wave-wide load brings eight rows: lane L lands at byte 16 L of the wave's 1 KB window (the
// hardware's rule), i.e. row L >> 3, position L & 7, so it fetches chunk (L & 7) ^ (L >> 3) of that row: eight
// neighbouring lanes cover one whole 128-byte line of global memory.  An operand read (lane = row li, chunk
// 4 s + kb) goes to position (4 s + kb) ^ (li & 7): the eight lanes of one pass hit eight different 16-byte bank
// groups.  Row offsets are 32-bit (the launcher checks that x and one expert's weights span less than 4 GB).
//
// Per 64-deep step: one block barrier (behind a wait for the wave's own loads of this stage: the stage is complete
// when every wave has passed), then the loads of the next step into the other stage, then 24 operand reads and 64
// MFMAs per wave.
// ---------------------------------------------------------------------------
// Wait until at most YOUNGER of the wave's loads are in flight (they complete in order) and its LDS reads are done,
// then the block barrier.  Written out: the fences of __syncthreads() make the compiler wait for every load in
// flight, the look-ahead ones included.
template <int YOUNGER>
__device__ __forceinline__ void loads_landed_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0x0070 | YOUNGER);  // vmcnt(YOUNGER) lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("" ::: "memory");
}
__device__ __forceinline__ void load16_to_lds(const bf16_t* base, uint32_t byte_offset, bf16_t* window) {
  __builtin_amdgcn_global_load_lds(
      (const __attribute__((address_space(1))) void*)(reinterpret_cast<const char*>(base) + byte_offset),
      (__attribute__((address_space(3))) void*)window, 16, 0, 0);
}

// 64 bits per lane from LDS, transposed among 16 lanes (ds_read_b64_tr_b16): with M[p][e] the four 16-bit elements
// e that lane p of a group of 16 points at, lane l receives M[4 e + (l >> 2)][l & 3], e = 0..3.
__device__ __forceinline__ uint2 lds_read_transposed(const char* p) {
  typedef short v4s __attribute__((ext_vector_type(4)));
  const v4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)p);
  return __builtin_bit_cast(uint2, v);
}

// TR = 1: the weight rows are input features (y = x W, the backward of TR = 0 on the same memory).  The weight
// tile of a step is then 64 rows of 256 outputs, 512 bytes a row, and lies in LDS as it lies in memory (a wave-wide
// load brings two rows; the 16-byte chunk c of row r at position c ^ ((r & 3) << 1)).  The MFMA operand, eight
// consecutive contraction indices of one output, is a column of that tile: two transposing LDS reads fetch it, each
// from four rows (which the swizzle puts on different banks) of 16 outputs.
template <int NKS, int TR>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void k_grouped_gemm_dl(
    GroupedArgs a, const GroupedPlanEntry* __restrict__ plan, const int32_t* __restrict__ nblocks,
    const int32_t* __restrict__ tile_group, const int32_t* __restrict__ slot_rows, int nsplit, int cpi) {
  constexpr int WN = 4, RB = 8, CB = 4, BM = 256, BN = 256;
  __shared__ __attribute__((aligned(1024))) bf16_t As0[BM * kGBK];
  __shared__ __attribute__((aligned(1024))) bf16_t As1[BM * kGBK];
  __shared__ __attribute__((aligned(1024))) bf16_t Bs0[BN * kGBK];
  __shared__ __attribute__((aligned(1024))) bf16_t Bs1[BN * kGBK];
  __shared__ __attribute__((aligned(1024))) bf16_t Bs2[BN * kGBK];
  const int blocks = *nblocks * nsplit;
  if ((int)blockIdx.x >= blocks) return;
  const int item = xcd_contiguous(blockIdx.x, blocks);
  const GroupedPlanEntry any = plan[item / nsplit];
  const int local = item - any.first * nsplit;
  const GroupedPlanEntry pe = plan[any.first + local % any.count];
  const int nb_first = (local / any.count) * cpi, nb_last = min(nb_first + cpi, a.N / BN);
  const int tid = threadIdx.x, lane = tid & 63, li = lane & 15, kb = lane >> 4;
  // (told to be uniform: the LDS windows of the wave's loads then live in scalar registers)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // The two strips of waves take the 16-row blocks of the tile alternately: strip wm owns rows 16 (2 rb + wm) + li,
  // rb = 0..7, i.e. half of every 32-row tile.  A block with fewer than eight tiles (the last of an expert) then
  // leaves both strips the same, smaller number of live row blocks, and its time shrinks with its rows.
  const int wm = wave / WN, wn = wave % WN;
  const int slot0 = pe.tile0 * kTileRows, live = pe.ntiles * kTileRows;

  // this wave's share of a stage: rows 32 wave + 8 i + (lane >> 3), i = 0..3, of the x tile and of the weight tile
  const int lrow = lane >> 3;
  const uint32_t lchunk = (uint32_t)(((lane & 7) ^ lrow) * 16);
  uint32_t xoff[4], woff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 32 * wave + 8 * i + lrow;
    int row = r < live ? slot_rows[slot0 + r] : -1;  // padding and dead rows read row 0 and are never stored
    row = min(max(row, 0), a.src_rows - 1);
    xoff[i] = (uint32_t)row * (uint32_t)(a.ldx * 2) + lchunk;
    if constexpr (TR) {
      const int kr = 8 * wave + 2 * i + (lane >> 5);  // row of the weight tile: two per load, 32 lanes each
      woff[i] = (uint32_t)kr * (uint32_t)(a.ldw * 2) + (uint32_t)(((lane & 31) ^ ((kr & 3) << 1)) * 16);
    } else {
      woff[i] = (uint32_t)r * (uint32_t)(a.ldw * 2) + lchunk;
    }
  }
  // operand reads: byte offsets inside a stage for s = 0, 1 (row block rb of the strip: + 4 KB rb, column block cb of
  // the wave: + 2 KB cb, as immediate offsets)
  uint32_t a_rd[2], b_rd[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    const uint32_t pos = (uint32_t)(((4 * s + kb) ^ (li & 7)) * 16);
    a_rd[s] = (uint32_t)(16 * wm + li) * 128u + pos;
    b_rd[s] = (uint32_t)(16 * CB * wn + li) * 128u + pos;
  }
  // TR: this lane's address in the weight tile for column block cb: row 8 kb + (li >> 2) (+ 32 s + 4 h as immediate
  // offsets), outputs 64 wn + 16 cb + 4 (li & 3) .. + 3
  uint32_t b_tr[CB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb)
    b_tr[cb] = (uint32_t)(8 * kb + (li >> 2)) * 512u +
               (uint32_t)((8 * wn + 2 * (cb ^ (li >> 2)) + ((li & 3) >> 1)) * 16 + (li & 1) * 8);
  const bf16_t* wbase = a.w + (int64_t)pe.expert * a.w_stride;
  const int nk = a.K / kGBK;
  const int window = (32 * wave) * kGBK;  // first element of this wave's rows in a stage

  for (int nb = nb_first; nb < nb_last; ++nb) {
    const bf16_t* wnb = TR ? wbase + nb * BN : wbase + (int64_t)nb * BN * a.ldw;
    f32x4 acc[RB][CB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) acc[rb][cb] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto fetch_x = [&](int ks, bf16_t* As) {
      const bf16_t* xk = a.x + ks * kGBK;
#pragma unroll
      for (int i = 0; i < 4; ++i) load16_to_lds(xk, xoff[i], As + window + 8 * i * kGBK);
    };
    auto fetch_w = [&](int ks, bf16_t* Bs) {
      if constexpr (TR) {
        const bf16_t* wk = wnb + (int64_t)ks * kGBK * a.ldw;
#pragma unroll
        for (int i = 0; i < 4; ++i) load16_to_lds(wk, woff[i], Bs + (8 * wave + 2 * i) * BN);
      } else {
        const bf16_t* wk = wnb + ks * kGBK;
#pragma unroll
        for (int i = 0; i < 4; ++i) load16_to_lds(wk, woff[i], Bs + window + 8 * i * kGBK);
      }
    };
    // One 64-deep step on NRB live row blocks per strip (NRB even).  In four quarters of 2 NRB MFMAs (half of the
    // row blocks of one 32-deep half step); the operand reads of a quarter are requested one quarter ahead, so
    // they land while the matrix cores work (the fences keep the compiler from moving them back next to their use).
    auto compute = [&](const bf16_t* As, const bf16_t* Bs, auto nrb_c) {
      constexpr int NRB = decltype(nrb_c)::value, H = NRB / 2;
      const char* Ab = reinterpret_cast<const char*>(As);
      const char* Bb = reinterpret_cast<const char*>(Bs);
      uint4 fw[2][CB], fx[2][H];
      auto read_w = [&](int s) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
          if constexpr (TR) {
            const uint2 lo = lds_read_transposed(Bb + b_tr[cb] + 16384 * s);
            const uint2 hi = lds_read_transposed(Bb + b_tr[cb] + 16384 * s + 2048);
            fw[s][cb] = make_uint4(lo.x, lo.y, hi.x, hi.y);
          } else {
            fw[s][cb] = *reinterpret_cast<const uint4*>(Bb + b_rd[s] + 2048 * cb);
          }
        }
      };
      auto read_x = [&](int s, int half) {
#pragma unroll
        for (int i = 0; i < H; ++i)
          fx[half][i] = *reinterpret_cast<const uint4*>(Ab + a_rd[s] + 4096 * (H * half + i));
      };
      auto quarter = [&](int s, int half) {
#pragma unroll
        for (int i = 0; i < H; ++i)
#pragma unroll
          for (int cb = 0; cb < CB; ++cb)
            acc[H * half + i][cb] = mfma16(fw[s][cb], fx[half][i], acc[H * half + i][cb]);
      };
      read_w(0);
      read_x(0, 0);
      read_x(0, 1);
      __builtin_amdgcn_sched_barrier(0);
      quarter(0, 0);
      __builtin_amdgcn_sched_barrier(0);
      read_w(1);
      read_x(1, 0);
      __builtin_amdgcn_sched_barrier(0);
      quarter(0, 1);
      __builtin_amdgcn_sched_barrier(0);
      read_x(1, 1);
      __builtin_amdgcn_sched_barrier(0);
      quarter(1, 0);
      quarter(1, 1);
      __builtin_amdgcn_sched_barrier(0);
    };
    // The weight tiles, most of which come from memory, are requested two steps ahead (three stages), the x tiles,
    // most of which another column block of the same rows has just brought into this XCD's L2, one step ahead (two
    // stages).  Step ks: wait until of the wave's loads only the youngest four (the weight tile of step ks + 1) may
    // still be in flight, block barrier (x and weight tile of step ks are complete, the stages of step ks - 1 have
    // been read by everybody), request x of step ks + 1 and the weights of step ks + 2, compute.
    // (Every step requests both tiles, past the last step the last ones again, into stages that are not read any
    // more: the same count of loads in flight at every barrier, and no branch in the steady state.)
    auto stage_a = [&](auto i) -> bf16_t* {
      if constexpr (decltype(i)::value == 0) return As0;
      else return As1;
    };
    auto stage_b = [&](auto i) -> bf16_t* {
      if constexpr (decltype(i)::value == 0) return Bs0;
      else if constexpr (decltype(i)::value == 1) return Bs1;
      else return Bs2;
    };
    auto step = [&](int ks, auto phase, auto nrb_c) {  // phase = ks mod 6
      constexpr int P = decltype(phase)::value;
      loads_landed_barrier<4>();
      fetch_x(min(ks + 1, nk - 1), stage_a(std::integral_constant<int, (P + 1) % 2>{}));
      fetch_w(min(ks + 2, nk - 1), stage_b(std::integral_constant<int, (P + 2) % 3>{}));
      compute(stage_a(std::integral_constant<int, P % 2>{}), stage_b(std::integral_constant<int, P % 3>{}), nrb_c);
    };
    auto k_loop = [&](auto nrb_c) {
      fetch_x(0, As0);
      fetch_w(0, Bs0);
      fetch_w(min(1, nk - 1), Bs1);
      int ks = 0;
      using std::integral_constant;
      for (; ks + 6 <= nk; ks += 6) {
        step(ks, integral_constant<int, 0>{}, nrb_c);
        step(ks + 1, integral_constant<int, 1>{}, nrb_c);
        step(ks + 2, integral_constant<int, 2>{}, nrb_c);
        step(ks + 3, integral_constant<int, 3>{}, nrb_c);
        step(ks + 4, integral_constant<int, 4>{}, nrb_c);
        step(ks + 5, integral_constant<int, 5>{}, nrb_c);
      }
      if (ks < nk) step(ks, integral_constant<int, 0>{}, nrb_c);
      if (ks + 1 < nk) step(ks + 1, integral_constant<int, 1>{}, nrb_c);
      if (ks + 2 < nk) step(ks + 2, integral_constant<int, 2>{}, nrb_c);
      if (ks + 3 < nk) step(ks + 3, integral_constant<int, 3>{}, nrb_c);
      if (ks + 4 < nk) step(ks + 4, integral_constant<int, 4>{}, nrb_c);
      loads_landed_barrier<0>();  // every stage has been read, no load is in flight: the next column block may load
    };
    // live row blocks per strip = tiles of the block, rounded up to even (dead rows hold row 0 of x: their sums are
    // never stored)
    if (pe.ntiles > 6) k_loop(std::integral_constant<int, 8>{});
    else if (pe.ntiles > 4) k_loop(std::integral_constant<int, 6>{});
    else if (pe.ntiles > 2) k_loop(std::integral_constant<int, 4>{});
    else k_loop(std::integral_constant<int, 2>{});

    if constexpr (NKS > 0) {
      // LoRA term: h[slot][0 .. rpad) against B_g[n][0 .. rank); row block rb of a strip lies in tile rb of the
      // block (a tile has one group)
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if (rb >= pe.ntiles) break;
        const int g = checked_group(tile_group[pe.tile0 + rb], a.tb);
        const int r = g >= 0 ? min(a.rank[g], a.rpad) : 0;
        if (r <= 0) continue;
        const bf16_t* Bg = (const bf16_t*)a.lora_B[g];
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
          const int n0 = 32 * s + 8 * kb;  // first rank index of this lane's operand piece
          if (32 * s >= r) break;          // uniform over the wave
          const int slot = slot0 + 32 * rb + 16 * wm + li;
          const uint4 fh = n0 < a.rpad ? ld16(a.hrow + (int64_t)slot * a.rpad + n0) : zero4();
          uint4 fb[CB];
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) {
            const int n = nb * BN + 16 * CB * wn + 16 * cb + li;
            fb[cb] = n0 < r ? keep_first(ld16(Bg + (int64_t)n * a.ldb + n0), r - n0) : zero4();
          }
#pragma unroll
          for (int cb = 0; cb < CB; ++cb) acc[rb][cb] = mfma16(fb[cb], fh, acc[rb][cb]);
        }
      }
    }

    // lane holds y[slot 16 (2 rb + wm) + li][nb BN + 16 CB wn + 16 cb + 4 kb + v], v = 0..3: 8-byte stores
    // (the rows are looked up here, all eight together, rather than kept in registers across the loop)
    int out_row[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int r = 16 * (2 * rb + wm) + li;
      out_row[rb] = r < live ? checked_row(slot_rows[slot0 + r], a.tb) : -1;
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      if (out_row[rb] < 0) continue;
      bf16_t* yp = a.y + (int64_t)out_row[rb] * a.ldy + nb * BN + 16 * CB * wn + 4 * kb;
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        const f32x4 v = acc[rb][cb];
        *reinterpret_cast<uint2*>(yp + 16 * cb) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
      }
    }
  }
}

}  // namespace

bool grouped_gemm_supported(const GroupedArgs& a) {
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  if (a.K < kGBK || a.K % kGBK != 0 || a.N < 128 || a.N % 128 != 0) return false;
  if (a.ldx % 8 != 0 || a.ldw % 8 != 0 || a.w_stride % 8 != 0 || a.ldy % 4 != 0) return false;
  if (!al16(a.x) || !al16(a.w) || (reinterpret_cast<uintptr_t>(a.y) & 7u) != 0) return false;
  if (a.rpad != 0 && (a.rpad > 64 || a.ldb % 8 != 0 || !al16(a.hrow))) return false;
  return true;
}

// upper bound of the row blocks, for either block size (workspace sizing)
int64_t grouped_plan_entries(const SegLayout& L, int64_t experts) { return ceil_div(L.max_tiles, 4) + experts; }

int launch_grouped_gemm(const GroupedArgs& a, int experts, int nt, GroupedPlanEntry* plan, int32_t* nblocks,
                        const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  // The 8-wave variants win wherever they apply.  The forward form loads its tiles straight into LDS
  // (k_grouped_gemm_dl: 32-bit row offsets, so x and one expert's weights must span less than 4 GB); the older
  // 8-wave kernel serves the transposing form and the rest, except with the LoRA term on small experts (its epilogue
  // has no registers to spare: measured at 512 rows per expert, 4 waves are then 5 % faster).
  const int nks = a.rpad == 0 ? 0 : (a.rpad <= 32 ? 1 : 2);
  // (TK_GROUPED_DIRECT=0 in the environment keeps the register-staged kernels in use: an A/B switch, read per call)
  const char* env_direct = getenv("TK_GROUPED_DIRECT");
  const bool direct = TK_GROUPED_DL && !(env_direct && env_direct[0] == '0') &&
                      (int64_t)a.src_rows * a.ldx * 2 < (1ll << 32) &&
                      (int64_t)(a.w_rows_are_inputs ? a.K : a.N) * a.ldw * 2 < (1ll << 32);
  const bool big =
      TK_GROUPED_BIG && a.N % 256 == 0 && (nks == 0 || direct || L.rows >= (int64_t)1024 * experts);
  const int ptiles = big ? 8 : 4, bn = big ? 256 : 128;
  const int max_entries = (int)(ceil_div(L.max_tiles, ptiles) + experts);
  hipLaunchKernelGGL(k_grouped_plan, dim3(1), dim3(256), 0, s, seg.tile_first, experts, nt, plan, nblocks, max_entries,
                     ptiles, (int)L.max_tiles);
  const int32_t* rows = seg.slot_table(a.map_rows);
  // several thousand work items, so that the last round of blocks on the 256 CUs is a small part of the run
  const int ncb = a.N / bn;
  const int64_t row_blocks = ceil_div(L.max_tiles, ptiles);
  const int cpi = (int)std::min<int64_t>(ncb, std::max<int64_t>(1, ceil_div(ncb * row_blocks, kGroupedItems)));
  const int nsplit = (int)ceil_div(ncb, cpi);
  const dim3 grid((unsigned)((int64_t)max_entries * nsplit));
#define TK_LAUNCH_GROUPED(NKS, BIG)                                                                                  \
  hipLaunchKernelGGL((k_grouped_gemm<NKS, BIG, 0>), grid, dim3(BIG ? 512 : 256), 0, s, a, plan, nblocks, seg.tile_group, \
                     rows, nsplit, cpi)
  if (a.w_rows_are_inputs && big && direct) {  // never with the LoRA term (the caller checks)
    hipLaunchKernelGGL((k_grouped_gemm_dl<0, 1>), grid, dim3(512), 0, s, a, plan, nblocks, seg.tile_group, rows, nsplit,
                       cpi);
  } else if (a.w_rows_are_inputs) {
    if (big)
      hipLaunchKernelGGL((k_grouped_gemm<0, 1, 1>), grid, dim3(512), 0, s, a, plan, nblocks, seg.tile_group, rows, nsplit,
                         cpi);
    else
      hipLaunchKernelGGL((k_grouped_gemm<0, 0, 1>), grid, dim3(256), 0, s, a, plan, nblocks, seg.tile_group, rows, nsplit,
                         cpi);
  } else if (big && direct) {
    if (nks == 0)
      hipLaunchKernelGGL((k_grouped_gemm_dl<0, 0>), grid, dim3(512), 0, s, a, plan, nblocks, seg.tile_group, rows, nsplit, cpi);
    else if (nks == 1)
      hipLaunchKernelGGL((k_grouped_gemm_dl<1, 0>), grid, dim3(512), 0, s, a, plan, nblocks, seg.tile_group, rows, nsplit, cpi);
    else
      hipLaunchKernelGGL((k_grouped_gemm_dl<2, 0>), grid, dim3(512), 0, s, a, plan, nblocks, seg.tile_group, rows, nsplit, cpi);
  } else if (big) {
    if (nks == 0) TK_LAUNCH_GROUPED(0, 1);
    else if (nks == 1) TK_LAUNCH_GROUPED(1, 1);
    else TK_LAUNCH_GROUPED(2, 1);
  } else {
    if (nks == 0) TK_LAUNCH_GROUPED(0, 0);
    else if (nks == 1) TK_LAUNCH_GROUPED(1, 0);
    else TK_LAUNCH_GROUPED(2, 0);
  }
#undef TK_LAUNCH_GROUPED
  return check_launch();
}

}  // namespace tk
