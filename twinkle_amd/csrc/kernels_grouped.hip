// Grouped base GEMM of packed experts with the LoRA term in its epilogue (gfx950, bf16 MFMA).
//
//   y[row(slot)][n] = sum_k x[row(slot)][k] * W_e[n][k]  (+ sum_r h[slot][r] * B_g[n][r])
//
// for every slot of the segment table, e = g / groups_per_weight the weight (expert) of the slot's group g.
// One launch serves all experts: the reference loops over the experts on the host and synchronises for each
// chunk boundary.  The LoRA term enters as extra contraction steps on the accumulators, so y is written once
// instead of written by the GEMM and then read, updated and written again by the expand kernel.
//
//   k_grouped_plan   one small block: the list of row blocks (up to 4 consecutive tiles of one expert)
//   k_grouped_gemm   one block of 4 waves per row block, looping over the 128-column blocks of the output: the
//                    row block's x stays in L2 across the column blocks and the row blocks of one expert, which
//                    reach an XCD together, stream that expert's weights through the XCD's L2 side by side
//
// Block tile 128 x 128 x 64, double-buffered in LDS (row stride 144 B: conflict-free 16-byte operand reads), a
// wave owns 64 x 64 as 4 x 4 MFMA 16x16x32 tiles.  The weight fragment is the MFMA A operand and the x fragment
// the B operand, so a lane ends up with four consecutive output columns of one row.
#include <algorithm>
#include <type_traits>

#include "tk_mfma.h"

namespace tk {

namespace {

constexpr int kGBM = 128, kGBN = 128, kGBK = 64, kGLS = kGBK + 8;
constexpr int kPlanTiles = kGBM / kTileRows;  // tiles per row block
#ifndef TK_GROUPED_ITEMS
#define TK_GROUPED_ITEMS 6144
#endif
constexpr int kGroupedItems = TK_GROUPED_ITEMS;  // work items aimed at per launch

__global__ __launch_bounds__(256) void k_grouped_plan(const int32_t* __restrict__ tile_first, int experts, int nt,
                                                      GroupedPlanEntry* __restrict__ plan,
                                                      int32_t* __restrict__ nblocks, int max_entries) {
  __shared__ int32_t sums[256];
  const int tid = threadIdx.x;
  const int per = (experts + 255) / 256;
  const int e0 = min(experts, tid * per), e1 = min(experts, e0 + per);
  int cnt = 0;
  for (int e = e0; e < e1; ++e)
    cnt += (tile_first[(e + 1) * nt] - tile_first[e * nt] + kPlanTiles - 1) / kPlanTiles;
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
    const int t0 = tile_first[e * nt], t1 = tile_first[(e + 1) * nt];
    const int first = at, count = (t1 - t0 + kPlanTiles - 1) / kPlanTiles;
    for (int t = t0; t < t1; t += kPlanTiles, ++at)
      if (at < max_entries) plan[at] = GroupedPlanEntry{t, min(kPlanTiles, t1 - t), e, first, count, 0};
  }
  if (tid == 255) *nblocks = min(sums[255], max_entries);
}

// NKS: MFMA steps of the LoRA term (0: none; 1: padded rank 16 or 32; 2: padded rank 64)
template <int NKS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void k_grouped_gemm(GroupedArgs a, const GroupedPlanEntry* __restrict__ plan,
                                                      const int32_t* __restrict__ nblocks,
                                                      const int32_t* __restrict__ tile_group,
                                                      const int32_t* __restrict__ slot_rows, int nsplit, int cpi) {
  __shared__ __attribute__((aligned(16))) bf16_t As[2][kGBM * kGLS];  // x rows
  __shared__ __attribute__((aligned(16))) bf16_t Bs[2][kGBN * kGLS];  // weight rows
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
  const int nb_first = (local / any.count) * cpi, nb_last = min(nb_first + cpi, a.N / kGBN);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;
  const int slot0 = pe.tile0 * kTileRows, live = pe.ntiles * kTileRows;

  // global -> LDS: thread t moves 16 bytes of rows (t >> 3) + 32 i, i = 0..3, at column chunk t & 7
  const int lrow = tid >> 3, lchunk = (tid & 7) * 8;
  const bf16_t* xp[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = lrow + 32 * i;
    int row = r < live ? slot_rows[slot0 + r] : -1;  // padding and dead rows read row 0 and are never stored
    row = min(max(row, 0), a.src_rows - 1);
    xp[i] = a.x + (int64_t)row * a.ldx + lchunk;
  }
  // rows this lane stores: slots 64 wm + 16 rb + li
  int out_row[4];
#pragma unroll
  for (int rb = 0; rb < 4; ++rb) {
    const int r = 64 * wm + 16 * rb + li;
    out_row[rb] = r < live ? slot_rows[slot0 + r] : -1;
  }
  const bf16_t* wbase = a.w + (int64_t)pe.expert * a.w_stride;
  const int nk = a.K / kGBK;
  const int ldsw = lrow * kGLS + lchunk;  // + 32 i rows

  for (int nb = nb_first; nb < nb_last; ++nb) {
    const bf16_t* wp[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) wp[i] = wbase + (int64_t)(nb * kGBN + lrow + 32 * i) * a.ldw + lchunk;
    f32x4 acc[4][4];
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) acc[rb][cb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Two register sets: the loads of step ks + 2 are issued before step ks is computed and wait in registers
    // across one barrier (which orders LDS traffic only), so a load has two steps of MFMA work to arrive.
    uint4 gx[2][4], gw[2][4];
    auto fetch = [&](int ks, auto set) {
      const int k0 = ks * kGBK;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        gx[set][i] = ld16(xp[i] + k0);
        gw[set][i] = ld16(wp[i] + k0);
      }
    };
    auto stash = [&](int buf, auto set) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        st16(&As[buf][ldsw + 32 * i * kGLS], gx[set][i]);
        st16(&Bs[buf][ldsw + 32 * i * kGLS], gw[set][i]);
      }
    };
    auto step = [&](int ks, auto parity) {  // parity = ks & 1 as a compile-time constant
      constexpr int cur = decltype(parity)::value;
      if (ks + 2 < nk) fetch(ks + 2, std::integral_constant<int, cur>{});
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        uint4 fx[4], fw[4];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) fx[rb] = ld16(&As[cur][(64 * wm + 16 * rb + li) * kGLS + 32 * s + 8 * kb]);
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) fw[cb] = ld16(&Bs[cur][(64 * wn + 16 * cb + li) * kGLS + 32 * s + 8 * kb]);
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
          for (int cb = 0; cb < 4; ++cb) acc[rb][cb] = mfma16(fw[cb], fx[rb], acc[rb][cb]);
      }
      if (ks + 1 < nk) stash(cur ^ 1, std::integral_constant<int, cur ^ 1>{});
      lds_barrier();
    };
    fetch(0, std::integral_constant<int, 0>{});
    if (nk > 1) fetch(1, std::integral_constant<int, 1>{});
    stash(0, std::integral_constant<int, 0>{});
    lds_barrier();
    for (int ks = 0; ks < nk; ks += 2) {
      step(ks, std::integral_constant<int, 0>{});
      if (ks + 1 < nk) step(ks + 1, std::integral_constant<int, 1>{});
    }

    if constexpr (NKS > 0) {
      // LoRA term: h[slot][0 .. rpad) against B_g[n][0 .. rank), per 32-row tile (a tile has one group)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int tile = pe.tile0 + 2 * wm + half;
        if (2 * wm + half >= pe.ntiles) break;
        const int g = tile_group[tile];
        const int r = g >= 0 ? min(a.rank[g], a.rpad) : 0;
        if (r <= 0) continue;
        const bf16_t* Bg = (const bf16_t*)a.lora_B[g];
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
          const int n0 = 32 * s + 8 * kb;  // first rank index of this lane's operand piece
          if (32 * s >= r) break;          // uniform over the wave
          uint4 fh[2], fb[4];
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const int slot = slot0 + 64 * wm + 32 * half + 16 * q + li;
            fh[q] = n0 < a.rpad ? ld16(a.hrow + (int64_t)slot * a.rpad + n0) : zero4();
          }
#pragma unroll
          for (int cb = 0; cb < 4; ++cb) {
            const int n = nb * kGBN + 64 * wn + 16 * cb + li;
            fb[cb] = n0 < r ? keep_first(ld16(Bg + (int64_t)n * a.ldb + n0), r - n0) : zero4();
          }
#pragma unroll
          for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int cb = 0; cb < 4; ++cb) acc[2 * half + q][cb] = mfma16(fb[cb], fh[q], acc[2 * half + q][cb]);
        }
      }
    }

    // lane holds y[slot 64 wm + 16 rb + li][nb 128 + 64 wn + 16 cb + 4 kb + v], v = 0..3: 8-byte stores
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      if (out_row[rb] < 0) continue;
      bf16_t* yp = a.y + (int64_t)out_row[rb] * a.ldy + nb * kGBN + 64 * wn + 4 * kb;
#pragma unroll
      for (int cb = 0; cb < 4; ++cb) {
        const f32x4 v = acc[rb][cb];
        *reinterpret_cast<uint2*>(yp + 16 * cb) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
      }
    }
  }
}

}  // namespace

bool grouped_gemm_supported(const GroupedArgs& a) {
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  if (a.K < kGBK || a.K % kGBK != 0 || a.N < kGBN || a.N % kGBN != 0) return false;
  if (a.ldx % 8 != 0 || a.ldw % 8 != 0 || a.w_stride % 8 != 0 || a.ldy % 4 != 0) return false;
  if (!al16(a.x) || !al16(a.w) || (reinterpret_cast<uintptr_t>(a.y) & 7u) != 0) return false;
  if (a.rpad != 0 && (a.rpad > 64 || a.ldb % 8 != 0 || !al16(a.hrow))) return false;
  return true;
}

int64_t grouped_plan_entries(const SegLayout& L, int64_t experts) { return ceil_div(L.max_tiles, kPlanTiles) + experts; }

int launch_grouped_gemm(const GroupedArgs& a, int experts, int nt, GroupedPlanEntry* plan, int32_t* nblocks,
                        const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (L.rows == 0) return TK_OK;
  const int max_entries = (int)grouped_plan_entries(L, experts);
  hipLaunchKernelGGL(k_grouped_plan, dim3(1), dim3(256), 0, s, seg.tile_first, experts, nt, plan, nblocks, max_entries);
  const int32_t* rows = seg.slot_table(a.map_rows);
  // several thousand work items, so that the last round of blocks on the 256 CUs is a small part of the run
  const int ncb = a.N / kGBN;
  const int64_t row_blocks = ceil_div(L.max_tiles, kPlanTiles);
  const int cpi = (int)std::min<int64_t>(ncb, std::max<int64_t>(1, ceil_div(ncb * row_blocks, kGroupedItems)));
  const int nsplit = (int)ceil_div(ncb, cpi);
  const dim3 grid((unsigned)((int64_t)max_entries * nsplit));
  if (a.rpad == 0)
    hipLaunchKernelGGL(k_grouped_gemm<0>, grid, dim3(256), 0, s, a, plan, nblocks, seg.tile_group, rows, nsplit, cpi);
  else if (a.rpad <= 32)
    hipLaunchKernelGGL(k_grouped_gemm<1>, grid, dim3(256), 0, s, a, plan, nblocks, seg.tile_group, rows, nsplit, cpi);
  else
    hipLaunchKernelGGL(k_grouped_gemm<2>, grid, dim3(256), 0, s, a, plan, nblocks, seg.tile_group, rows, nsplit, cpi);
  return check_launch();
}

}  // namespace tk
