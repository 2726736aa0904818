// Segment builder (stable counting sort of rows by group) and the row
// gather / scatter-back kernels that use its table.  Integer work, HBM-light:
// the table is built once per batch and read by every LoRA layer.
//
// Small inputs take one launch (k_seg_one, below).  General pipeline (three
// launches, no host synchronisation anywhere):
//   k_seg_hist    one wave per 512 rows: per-key counts by bit-sliced ballots
//                 (no contended atomics) -> hist[block][group]
//   k_seg_scan    one block: per-group totals, exclusive scans -> offsets and
//                 the firsts of the tile / chunk / partial tables, per-block
//                 bases (in place in hist); then, in parallel over tiles and
//                 slots, tile_group, the chunk table, slot_pos and the -1
//                 padding of slot_row
//   k_seg_scatter one wave per 512 rows: stable rank inside the wave by
//                 bit-sliced ballots, cursor per group in LDS -> inv, slot_row
#include <initializer_list>

#include "tk_device.h"

namespace tk {

namespace {

constexpr int kKeysPerLane = kSortBlockRows / 64;

// The kernels below sort into `buckets` = groups + 1 buckets: a key outside [0, groups) (a padding row, a row
// the caller marks with -1) goes to the last bucket, whose tiles and chunks carry group -1, so that such rows
// belong to no adapter: they keep their place in the permutation (after every group) and nothing else.
template <typename KeyT>
__device__ inline int load_key(const KeyT* keys, int64_t f, int buckets, int* bad) {
  long long k = (long long)keys[f];
  if (k < 0 || k >= buckets - 1) {
    *bad += 1;
    k = buckets - 1;
  }
  return (int)k;
}

// Eight consecutive keys starting at row f0 (a multiple of 8), as 16-byte loads where the array allows;
// rows past the end give -1.
template <typename KeyT>
__device__ inline void load_keys8(const KeyT* keys, int64_t f0, int64_t rows, bool aligned16, int buckets, int* bad,
                                  int (&out)[8]) {
  if (aligned16 && f0 + 8 <= rows) {
    long long raw[8];
    if constexpr (sizeof(KeyT) == 4) {
      const int4 a = *reinterpret_cast<const int4*>(keys + f0), b = *reinterpret_cast<const int4*>(keys + f0 + 4);
      const int v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) raw[j] = v[j];
    } else {
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        const longlong2 a = *reinterpret_cast<const longlong2*>(keys + f0 + j);
        raw[j] = a.x;
        raw[j + 1] = a.y;
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool off = raw[j] < 0 || raw[j] >= buckets - 1;
      *bad += off;
      out[j] = off ? buckets - 1 : (int)raw[j];
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) out[j] = f0 + j < rows ? load_key(keys, f0 + j, buckets, bad) : -1;
}

// lanes of this wave that are valid and hold the same key as the calling lane
__device__ inline unsigned long long same_key_lanes(bool valid, int key, int key_bits) {
  unsigned long long same = __ballot(valid);
  for (int b = 0; b < key_bits; ++b) {
    const bool bit = (key >> b) & 1;
    const unsigned long long m = __ballot(valid && bit);
    same &= bit ? m : ~m;
  }
  return same;
}

template <typename KeyT>
__global__ __launch_bounds__(64) void k_seg_hist(const KeyT* __restrict__ keys, int rows, int groups, int key_bits,
                                                 int32_t* __restrict__ hist, int32_t* __restrict__ bad_out) {
  extern __shared__ int32_t lds[];
  const int lane = threadIdx.x;
  const int blk = blockIdx.x;
  for (int g = lane; g < groups; g += 64) lds[g] = 0;
  __syncthreads();
  int bad = 0;
  const int64_t base = (int64_t)blk * kSortBlockRows;
  int k[kKeysPerLane];
#pragma unroll
  for (int j = 0; j < kKeysPerLane; ++j) {  // all loads first: they overlap
    const int64_t f = base + j * 64 + lane;
    k[j] = f < rows ? load_key(keys, f, groups, &bad) : -1;
  }
#pragma unroll
  for (int j = 0; j < kKeysPerLane; ++j) {
    const bool valid = k[j] >= 0;
    const unsigned long long same = same_key_lanes(valid, k[j], key_bits);
    const bool leader = valid && (same & ((1ull << lane) - 1ull)) == 0;
    if (leader) lds[k[j]] += __popcll(same);  // one lane per distinct key: no conflicts
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();
  for (int g = lane; g < groups; g += 64) hist[(int64_t)blk * groups + g] = lds[g];
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) bad += __shfl_xor(bad, d, 64);
  if (lane == 0) bad_out[blk] = bad;
}

// Exclusive scan of one value per thread over a 1024-thread block.
__device__ inline int block_exclusive_scan(int v, int* wave_sums, int* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int o = __shfl_up(incl, d, 64);
    if (lane >= d) incl += o;
  }
  if (lane == 63) wave_sums[wave] = incl;
  __syncthreads();
  if (wave == 0) {
    int w = lane < 16 ? wave_sums[lane] : 0;
    int wi = w;
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) {
      int o = __shfl_up(wi, d, 64);
      if (lane >= d) wi += o;
    }
    if (lane < 16) wave_sums[lane] = wi - w;  // exclusive base of each wave
    if (lane == 15) wave_sums[16] = wi;        // block total
  }
  __syncthreads();
  const int res = wave_sums[wave] + incl - v;
  *total = wave_sums[16];
  __syncthreads();
  return res;
}

// largest g in [0, groups) with first[g] <= i, for a non-decreasing `first` with first[groups] > i
__device__ inline int group_of(const int32_t* first, int groups, int i) {
  int lo = 0, hi = groups;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (first[mid] <= i) lo = mid; else hi = mid;
  }
  return lo;
}

// Per-group prefix over the sort blocks' counts (each block's exclusive base inside its group), then the prefix over
// the groups: offsets, first tile, first chunk and first partial slot of every group, and the header.  One block; a
// thread owns a group and requests the counts of 32 sort blocks together: the chain over the sort blocks is what the
// kernel waits for (eight at a time it took 37 us at 128 sort blocks x 513 groups, 32 at a time 13.6 us; with 64 the
// registers of a 1024-thread block spill to 376 bytes of scratch memory per thread, and with that one kernel in it the
// whole step went from 442 to 597 us).  The per-tile and per-chunk tables are filled by extra blocks of the scatter
// launch that follows.
constexpr int kScanBatch = 32;

__global__ __launch_bounds__(1024) void k_seg_scan(int rows, int groups, int sort_blocks, SegView V, int chunk_tiles,
                                                   int64_t* __restrict__ offsets_out) {
  __shared__ int wave_sums[17];
  const int tid = threadIdx.x;
  int bad = 0;
  for (int b = tid; b < sort_blocks; b += 1024) bad += V.bad[b];
  int bad_total;
  block_exclusive_scan(bad, wave_sums, &bad_total);
  int carry_rows = 0, carry_tiles = 0, carry_chunks = 0, carry_part = 0;
  for (int g0 = 0; g0 < groups; g0 += 1024) {
    const int g = g0 + tid;
    int count = 0;
    if (g < groups) {
      for (int b0 = 0; b0 < sort_blocks; b0 += kScanBatch) {
        int c[kScanBatch];
#pragma unroll
        for (int j = 0; j < kScanBatch; ++j) c[j] = b0 + j < sort_blocks ? V.hist[(int64_t)(b0 + j) * groups + g] : 0;
#pragma unroll
        for (int j = 0; j < kScanBatch; ++j) {
          if (b0 + j < sort_blocks) V.hist[(int64_t)(b0 + j) * groups + g] = count;
          count += c[j];
        }
      }
    }
    const int ntile = (count + kTileRows - 1) / kTileRows;
    const int nchunk = (ntile + chunk_tiles - 1) / chunk_tiles;
    const int npart = (nchunk > 1 && g != groups - 1) ? nchunk : 0;  // rows without a group need no partials
    int tot;
    const int e_rows = block_exclusive_scan(count, wave_sums, &tot) + carry_rows;
    carry_rows += tot;
    const int e_tiles = block_exclusive_scan(ntile, wave_sums, &tot) + carry_tiles;
    carry_tiles += tot;
    const int e_chunks = block_exclusive_scan(nchunk, wave_sums, &tot) + carry_chunks;
    carry_chunks += tot;
    const int e_part = block_exclusive_scan(npart, wave_sums, &tot) + carry_part;
    carry_part += tot;
    if (g < groups) {
      V.offsets[g] = e_rows;
      V.tile_first[g] = e_tiles;
      V.chunk_first[g] = e_chunks;
      V.partial_first[g] = e_part;
      if (offsets_out) offsets_out[g] = e_rows;  // [groups - 1] (the caller's last entry): rows that have a group
    }
  }
  if (tid == 0) {
    V.offsets[groups] = carry_rows;
    V.tile_first[groups] = carry_tiles;
    V.chunk_first[groups] = carry_chunks;
    V.partial_first[groups] = carry_part;
    SegHeader* hdr = V.header;
    hdr->magic = kSegMagic;
    hdr->rows = rows;
    hdr->groups = groups - 1;
    hdr->num_tiles = carry_tiles;
    hdr->num_chunks = carry_chunks;
    hdr->num_partials = carry_part;
    hdr->bad_keys = bad_total;
    hdr->identity_order = 1;
  }
}

// Per-tile (with its 32 slots) and per-chunk entries of the table from the groups' firsts: entry i by thread i of the
// fill blocks (the blocks of the scatter launch past its sort blocks).  slot_row: only the padding is written here,
// the rows come from the scatter blocks.
__device__ inline void seg_fill_tables(const SegView& V, int groups, int max_tiles, int max_chunks, int chunk_tiles,
                                       int thread, int threads) {
  const int32_t* offs = V.offsets;
  const int32_t* tfirst = V.tile_first;
  const int32_t* cfirst = V.chunk_first;
  const int32_t* pfirst = V.partial_first;
  const int num_tiles = tfirst[groups], num_chunks = cfirst[groups];
  for (int i = thread; i < max_tiles; i += threads) {
    int g = -1, pos0 = 0, valid = 0;
    if (i < num_tiles) {
      g = group_of(tfirst, groups, i);
      pos0 = offs[g] + (i - tfirst[g]) * kTileRows;   // sorted position of the tile's first slot
      valid = min(kTileRows, offs[g + 1] - pos0);       // padding is at the end of a group's last tile
    }
    V.tile_group[i] = g == groups - 1 ? -1 : g;
    V.tile_order[i] = i;  // this path leaves the tiles in table order
    if (i % kSetTiles == 0) V.set_order[i / kSetTiles] = i / kSetTiles;
    int4* sp = reinterpret_cast<int4*>(V.slot_pos + (int64_t)i * kTileRows);
#pragma unroll
    for (int j = 0; j < kTileRows; j += 4)
      sp[j / 4] = make_int4(j < valid ? pos0 + j : -1, j + 1 < valid ? pos0 + j + 1 : -1,
                            j + 2 < valid ? pos0 + j + 2 : -1, j + 3 < valid ? pos0 + j + 3 : -1);
    for (int j = valid; j < kTileRows; ++j) V.slot_row[(int64_t)i * kTileRows + j] = -1;
  }
  for (int i = thread; i < max_chunks; i += threads) {
    ChunkInfo c{-1, 0, 0, -1};
    if (i < num_chunks) {
      const int g = group_of(cfirst, groups, i);
      const int j = i - cfirst[g];
      const int ntile = tfirst[g + 1] - tfirst[g];
      c.group = g == groups - 1 ? -1 : g;
      c.tile0 = tfirst[g] + j * chunk_tiles;
      c.ntiles = min(chunk_tiles, ntile - j * chunk_tiles);
      c.partial = (cfirst[g + 1] - cfirst[g] > 1 && g != groups - 1) ? pfirst[g] + j : -1;
    }
    V.chunks[i] = c;
  }
}

template <typename KeyT>
__global__ __launch_bounds__(64) void k_seg_scatter(const KeyT* __restrict__ keys, int rows, int groups, int key_bits,
                                                    SegView V, int64_t* __restrict__ perm_out, int sort_blocks,
                                                    int max_tiles, int max_chunks, int chunk_tiles) {
  extern __shared__ int32_t cursor[];
  const int lane = threadIdx.x;
  const int blk = blockIdx.x;
  if (blk >= sort_blocks) {  // the blocks past the sort blocks fill the per-tile and per-chunk tables
    seg_fill_tables(V, groups, max_tiles, max_chunks, chunk_tiles, (blk - sort_blocks) * 64 + lane,
                    ((int)gridDim.x - sort_blocks) * 64);
    return;
  }
  const int64_t base = (int64_t)blk * kSortBlockRows;
  int unused = 0;
  int k[kKeysPerLane];
#pragma unroll
  for (int j = 0; j < kKeysPerLane; ++j) {  // all loads first: they overlap
    const int64_t f = base + j * 64 + lane;
    k[j] = f < rows ? load_key(keys, f, groups, &unused) : -1;
  }
  for (int g = lane; g < groups; g += 64) cursor[g] = V.offsets[g] + V.hist[(int64_t)blk * groups + g];
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kKeysPerLane; ++j) {
    const int64_t f = base + j * 64 + lane;
    const bool valid = k[j] >= 0;
    const int key = max(k[j], 0);
    // rows with equal keys keep their lane order
    const unsigned long long same = same_key_lanes(valid, key, key_bits);
    const int rank = __popcll(same & ((1ull << lane) - 1ull));
    int pos = 0;
    if (valid) pos = cursor[key] + rank;
    __builtin_amdgcn_wave_barrier();
    if (valid && rank == 0) cursor[key] += __popcll(same);
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      V.inv[f] = pos;
      if (perm_out) perm_out[pos] = f;
      // padded slot = 32 * first tile of the group + position inside the group
      V.slot_row[V.tile_first[key] * kTileRows + (pos - V.offsets[key])] = (int32_t)f;
    }
  }
}

// ---------------------------------------------------------------------------
// Single-launch builder for the common small case (at most kOneGroups groups and kOneBlocks * 512
// rows, i.e. one micro-batch of tokens over a handful of adapters).  Three dependent launches cost
// more than the work itself there, so every block redundantly counts *all* keys (a few hundred KB,
// served from L2), which gives it the group totals and the number of equal keys ahead of its own 512
// rows without any communication.  Counting is one LDS add per key into one of 16 sub-histograms
// (lane % 16, rows of 65 words: equal keys of different lanes fall into different banks).  The
// block's own 512 rows are ranked by its first 8 waves, one 64-row round each: rank inside the round
// from bit-sliced ballots, rounds before it from a small per-round table.  All threads then fill
// the block's share of the tile / chunk tables.  Integer adds only: the result does not depend on
// the order in which the adds land.
// ---------------------------------------------------------------------------
constexpr int kOneGroups = 64;
constexpr int kOneBlocks = 64;
constexpr int kOneWaves = 16;
constexpr int kOneSubs = 16;
constexpr int kOneBatch = kOneBlocks / kOneWaves;  // sort blocks whose keys a wave requests together

template <typename KeyT>
__global__ __launch_bounds__(kOneWaves * 64) void k_seg_one(const KeyT* __restrict__ keys, int rows, int groups,
                                                            int key_bits, int sort_blocks, int max_tiles,
                                                            int max_chunks, int chunk_tiles, SegView V,
                                                            int64_t* __restrict__ perm_out,
                                                            int64_t* __restrict__ offsets_out) {
  __shared__ int32_t cnt[2][kOneSubs][kOneGroups + 1];  // keys ahead of this block / in it and after it
  __shared__ int32_t round_cnt[kKeysPerLane][kOneGroups];  // this block's keys per 64-row round
  __shared__ int32_t first[4][kOneGroups + 1];          // offsets, tile_first, chunk_first, partial_first
  __shared__ int32_t cursor[kOneGroups];                // sorted position of the block's first row of each group
  __shared__ int32_t ahead[kKeysPerLane][kOneGroups];   // rows of each group ahead of each 64-row round of the block
  __shared__ int32_t bad_s[kOneWaves];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, blk = blockIdx.x;
  const int64_t base = (int64_t)blk * kSortBlockRows;

  // all key loads first: the block's own rows (one round per wave), then this wave's share of all rows
  int unused = 0, bad = 0;
  int mine = -1;
  if (wave < kKeysPerLane) {
    const int64_t f = base + wave * 64 + lane;
    mine = f < rows ? load_key(keys, f, groups, &unused) : -1;
  }
  // (which lane counts which key of a sort block is free: a lane takes eight neighbours)
  static_assert(kKeysPerLane == 8, "a lane loads eight consecutive keys of a sort block");
  const bool aligned16 = (reinterpret_cast<uintptr_t>(keys) & 15u) == 0;
  int k[kOneBatch][kKeysPerLane];
#pragma unroll
  for (int u = 0; u < kOneBatch; ++u)
    load_keys8(keys, (int64_t)(wave + u * kOneWaves) * kSortBlockRows + 8 * lane, rows, aligned16, groups, &bad, k[u]);
  for (int i = tid; i < 2 * kOneSubs * (kOneGroups + 1); i += kOneWaves * 64) (&cnt[0][0][0])[i] = 0;
  for (int i = tid; i < kKeysPerLane * kOneGroups; i += kOneWaves * 64) (&round_cnt[0][0])[i] = 0;
  __syncthreads();

#pragma unroll
  for (int u = 0; u < kOneBatch; ++u) {
    if (wave + u * kOneWaves >= sort_blocks) break;  // wave-uniform
    int32_t* c = cnt[wave + u * kOneWaves < blk ? 0 : 1][lane & (kOneSubs - 1)];
#pragma unroll
    for (int j = 0; j < kKeysPerLane; ++j)
      if (k[u][j] >= 0) atomicAdd(&c[k[u][j]], 1);
  }
  int rank_in_round = 0;
  if (wave < kKeysPerLane) {
    const bool valid = mine >= 0;
    const unsigned long long same = same_key_lanes(valid, max(mine, 0), key_bits);
    rank_in_round = __popcll(same & ((1ull << lane) - 1ull));  // rows with equal keys keep their lane order
    if (valid && rank_in_round == 0) round_cnt[wave][mine] = __popcll(same);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) bad += __shfl_xor(bad, d, 64);
  if (lane == 0) bad_s[wave] = bad;
  __syncthreads();

  if (wave == 0) {
    int before = 0, rest = 0;
    if (lane < groups) {
#pragma unroll
      for (int sub = 0; sub < kOneSubs; ++sub) {
        before += cnt[0][sub][lane];
        rest += cnt[1][sub][lane];
      }
    }
    const int count = before + rest;
    const int ntile = (count + kTileRows - 1) / kTileRows;
    const int nchunk = (ntile + chunk_tiles - 1) / chunk_tiles;
    const int npart = (nchunk > 1 && lane != groups - 1) ? nchunk : 0;
    int v[4] = {count, ntile, nchunk, npart}, excl[4], total[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      int incl = v[t];
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
      }
      excl[t] = incl - v[t];
      total[t] = __shfl(incl, 63, 64);
    }
    if (lane < groups) {
#pragma unroll
      for (int t = 0; t < 4; ++t) first[t][lane] = excl[t];
      cursor[lane] = excl[0] + before;
    }
    if (lane == 0) {
#pragma unroll
      for (int t = 0; t < 4; ++t) first[t][groups] = total[t];
    }
    if (blk == 0) {
      if (lane < groups) {
        V.offsets[lane] = excl[0];
        V.tile_first[lane] = excl[1];
        V.chunk_first[lane] = excl[2];
        V.partial_first[lane] = excl[3];
        if (offsets_out) offsets_out[lane] = excl[0];
      }
      if (lane == 0) {
        V.offsets[groups] = total[0];
        V.tile_first[groups] = total[1];
        V.chunk_first[groups] = total[2];
        V.partial_first[groups] = total[3];
        int bad_total = 0;
        for (int w = 0; w < kOneWaves; ++w) bad_total += bad_s[w];
        SegHeader* hdr = V.header;
        hdr->magic = kSegMagic;
        hdr->rows = rows;
        hdr->groups = groups - 1;
        hdr->num_tiles = total[1];
        hdr->num_chunks = total[2];
        hdr->num_partials = total[3];
        hdr->bad_keys = bad_total;
        hdr->identity_order = 0;
      }
    }
  }
  __syncthreads();

  const int32_t* offs = first[0];
  const int32_t* tfirst = first[1];
  const int32_t* cfirst = first[2];
  const int32_t* pfirst = first[3];
  // rows of every group ahead of every round: blocks before this one, then the rounds before it
  for (int i = tid; i < kKeysPerLane * groups; i += kOneWaves * 64) {
    const int w = i / groups, g2 = i - w * groups;
    int n = cursor[g2] - offs[g2];
    for (int w2 = 0; w2 < w; ++w2) n += round_cnt[w2][g2];
    ahead[w][g2] = n;
  }
  __syncthreads();
  if (wave < kKeysPerLane) {
    const int64_t f = base + wave * 64 + lane;
    const bool valid = mine >= 0;
    int in_group = 0;  // position of this row inside its group
    bool moved = false;
    if (valid) {
      in_group = ahead[wave][mine] + rank_in_round;
      const int pos = offs[mine] + in_group;
      moved = pos != f;
      V.inv[f] = pos;
      if (perm_out) perm_out[pos] = f;
      // padded slot = 32 * first tile of the group + position inside the group
      V.slot_row[tfirst[mine] * kTileRows + in_group] = (int32_t)f;
    }
    // Sweep order of the tiles.  The row that opens a tile (position inside its group a multiple of 32) knows how
    // many tiles open before it: for every group, the rows of that group ahead of this row, in units of 32, rounded
    // up.  Those counts are all here (blocks and rounds before this one from the table above, lanes before this
    // one from a ballot per group), so the tile's place in the order needs no sort and no second launch.
    // No row of the round moved in any round <=> the keys came in order <=> that order is the identity.
    const unsigned long long any_moved = __ballot(moved);
    if (lane == 0) V.round_moved[blk * kKeysPerLane + wave] = any_moved != 0ull;
    const bool opens = valid && mine != groups - 1 && (in_group & (kTileRows - 1)) == 0;
    if (__ballot(opens)) {  // wave-uniform
      // The same count over sets of kSetTiles tiles, for the tiles that open a set: of the tiles t0 .. t0 + n - 1 of a
      // group ahead, ceil((t0 + n) / kSetTiles) - ceil(t0 / kSetTiles) open one.
      // Lane g2 holds the figures of group g2 (at most 64 groups here); the loop reads them lane by lane.
      static_assert(kOneGroups <= 64, "one lane per group");
      const int gl = min(lane, groups - 1);
      const int ahead_up = ahead[wave][gl] + kTileRows - 1;  // rounds the tile count up
      const int first_up = tfirst[gl] + kSetTiles - 1;
      int place = 0, set_place = 0;
      for (int g2 = 0; g2 < groups - 1; ++g2) {
        const unsigned long long in_g2 = __ballot(mine == g2);
        // rows of the group ahead of this row: earlier rounds and blocks, and the lanes below this one
        const unsigned n_up = __builtin_amdgcn_mbcnt_hi(
            (unsigned)(in_g2 >> 32),
            __builtin_amdgcn_mbcnt_lo((unsigned)in_g2, (unsigned)__builtin_amdgcn_readlane(ahead_up, g2)));
        const unsigned tiles_ahead = n_up / kTileRows;
        const unsigned t0_up = (unsigned)__builtin_amdgcn_readlane(first_up, g2);
        place += tiles_ahead;
        set_place += (t0_up + tiles_ahead) / kSetTiles - t0_up / kSetTiles;
      }
      if (opens) {
        const int tile = tfirst[mine] + in_group / kTileRows;
        V.tile_order[place] = tile;
        if (tile % kSetTiles == 0) V.set_order[set_place] = tile / kSetTiles;
      }
    }
  }

  const int num_tiles = tfirst[groups], num_chunks = cfirst[groups];
  const int real_tiles = tfirst[groups - 1];  // the tiles of the rows without a group come after them
  // spread over the blocks: entry i belongs to thread i / sort_blocks of block i % sort_blocks
  const int stride = sort_blocks * kOneWaves * 64;
  for (int i = tid * sort_blocks + blk; i < max_tiles; i += stride) {
    int g = -1, pos0 = 0, valid = 0;
    if (i < num_tiles) {
      g = group_of(tfirst, groups, i);
      pos0 = offs[g] + (i - tfirst[g]) * kTileRows;  // sorted position of the tile's first slot
      valid = min(kTileRows, offs[g + 1] - pos0);      // padding is at the end of a group's last tile
    }
    V.tile_group[i] = g == groups - 1 ? -1 : g;
    if (i >= real_tiles) V.tile_order[i] = i;  // nothing to do in these: they stay where they are, after the others
    if (i >= real_tiles && i % kSetTiles == 0) V.set_order[i / kSetTiles] = i / kSetTiles;
    int4* sp = reinterpret_cast<int4*>(V.slot_pos + (int64_t)i * kTileRows);
#pragma unroll
    for (int j = 0; j < kTileRows; j += 4)
      sp[j / 4] = make_int4(j < valid ? pos0 + j : -1, j + 1 < valid ? pos0 + j + 1 : -1,
                            j + 2 < valid ? pos0 + j + 2 : -1, j + 3 < valid ? pos0 + j + 3 : -1);
    for (int j = valid; j < kTileRows; ++j) V.slot_row[(int64_t)i * kTileRows + j] = -1;
  }
  for (int i = tid * sort_blocks + blk; i < max_chunks; i += stride) {
    ChunkInfo c{-1, 0, 0, -1};
    if (i < num_chunks) {
      const int g = group_of(cfirst, groups, i);
      const int j = i - cfirst[g];
      const int ntile = tfirst[g + 1] - tfirst[g];
      c.group = g == groups - 1 ? -1 : g;
      c.tile0 = tfirst[g] + j * chunk_tiles;
      c.ntiles = min(chunk_tiles, ntile - j * chunk_tiles);
      c.partial = (cfirst[g + 1] - cfirst[g] > 1 && g != groups - 1) ? pfirst[g] + j : -1;
    }
    V.chunks[i] = c;
  }
}

// ---------------------------------------------------------------------------
// Work lists of the rank classes of one call (see WorkList): block (list, class) walks the items of its kind in the
// order the consumer wants them (tiles and sets of four tiles in sweep order when rows are gathered, everything else
// as numbered) and keeps those that hold a tile (a chunk) of a group whose rank lies in the class.  A stream
// compaction with a block-wide scan per 1024 items: the lists are dense, ordered, and the same on every run.
// ---------------------------------------------------------------------------
struct ClassListArgs {
  const int32_t* rank;
  int32_t n, map_rows;
  int32_t lo[kMaxClasses], hi[kMaxClasses];
  char* base[kMaxClasses];
};

__global__ __launch_bounds__(1024) void k_class_lists(ClassListArgs p, ClassListLayout CL, SegView V, int max_tiles,
                                                      int max_chunks) {
  __shared__ int wave_sums[17];
  const int which = blockIdx.x, c = blockIdx.y, tid = threadIdx.x;
  const int lo = p.lo[c], hi = p.hi[c];
  int32_t* out = (int32_t*)(p.base[c] + CL.off[which]);
  const int n_items = (int)CL.items[which];
  const int unit = which == kListTiles ? 1 : which == kListPairs ? 2 : which == kListOcts ? 8 : kSetTiles;
  const int32_t* order = nullptr;
  if (p.map_rows && which == kListTiles) order = V.tile_order;
  if (p.map_rows && which == kListSets) order = V.set_order;
  int running = 0;
  for (int base = 0; base < n_items; base += 1024) {
    const int i = base + tid;
    int id = 0, keep = 0;
    if (i < n_items) {
      id = order ? order[i] : i;
      if (which == kListChunks) {
        const int g = id < max_chunks ? V.chunks[id].group : -1;
        keep = g >= 0 && class_rank(p.rank[g], lo, hi) > 0;
      } else if (id >= 0 && id < n_items) {  // (an order entry is an item number; checked all the same)
        for (int u = 0; u < unit; ++u) {
          const int t = id * unit + u;
          const int g = t < max_tiles ? V.tile_group[t] : -1;
          keep |= g >= 0 && class_rank(p.rank[g], lo, hi) > 0;
        }
      }
    }
    int total;
    const int at = block_exclusive_scan(keep, wave_sums, &total);
    if (keep) out[running + at] = id;
    running += total;
  }
  if (tid == 0) ((int32_t*)p.base[c])[which] = running;
}

// 16 bytes of a row: the unit the row movers below load and store when width, strides and pointers allow
// (V = 8 bf16 / 4 fp32 elements), else V = 1.  The arithmetic per element and the order of every sum are the
// same for both.
template <typename T, int V>
struct alignas(V * sizeof(T)) RowVec {
  T v[V];
};

// dst[j] = src[perm[j] mod tokens] * w[token, k], one wave per padded slot (slot_row is perm in padded order)
template <typename T, int V>
__global__ __launch_bounds__(256) void k_permute(const T* __restrict__ src, int64_t ld_src, T* __restrict__ dst,
                                                 int64_t ld_dst, const T* __restrict__ w,
                                                 const int32_t* __restrict__ slot_row,
                                                 const int32_t* __restrict__ slot_pos, int tokens, int top_k,
                                                 int width, int slots) {
  const int slot = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (slot >= slots) return;
  const int f = slot_row[slot];
  const int j = slot_pos[slot];
  // (table entries are compared with the row count before they index: a row or position outside it is skipped)
  if (f < 0 || j < 0 || f >= tokens * top_k || j >= tokens * top_k) return;
  const int t = f % tokens, k = f / tokens;
  const RowVec<T, V>* s = reinterpret_cast<const RowVec<T, V>*>(src + (int64_t)t * ld_src);
  RowVec<T, V>* d = reinterpret_cast<RowVec<T, V>*>(dst + (int64_t)j * ld_dst);
  if (w) {
    const float wt = to_f32(w[(int64_t)t * top_k + k]);
    for (int c = lane; c < width / V; c += 64) {
      RowVec<T, V> x = s[c];
#pragma unroll
      for (int i = 0; i < V; ++i) from_f32(to_f32(x.v[i]) * wt, &x.v[i]);
      d[c] = x;
    }
  } else {
    for (int c = lane; c < width / V; c += 64) d[c] = s[c];
  }
}

// out[t] = sum_k rows[inv[k * tokens + t]] * w[t, k], k ascending, fp32 accumulation
template <typename T, int V>
__global__ __launch_bounds__(256) void k_unpermute(const T* __restrict__ rows_, int64_t ld_rows, T* __restrict__ out,
                                                   int64_t ld_out, const T* __restrict__ w,
                                                   const int32_t* __restrict__ inv, int tokens, int top_k, int width) {
  const int t = blockIdx.x;
  if (t >= tokens) return;
  for (int c = threadIdx.x; c < width / V; c += 256) {
    float acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = 0.f;
    for (int k = 0; k < top_k; ++k) {
      const int j = inv[(int64_t)k * tokens + t];
      if ((unsigned)j >= (unsigned)(tokens * top_k)) continue;  // (a position outside the table's rows adds nothing)
      const RowVec<T, V> x = reinterpret_cast<const RowVec<T, V>*>(rows_ + (int64_t)j * ld_rows)[c];
      const float wt = w ? to_f32(w[(int64_t)t * top_k + k]) : 1.f;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        float v = to_f32(x.v[i]);
        if (w) {
          // the reference scales the row in the activation dtype before adding (ep_utils.py:142)
          T r;
          from_f32(v * wt, &r);
          v = to_f32(r);
        }
        acc[i] += v;
      }
    }
    RowVec<T, V> o;
#pragma unroll
    for (int i = 0; i < V; ++i) from_f32(acc[i], &o.v[i]);
    reinterpret_cast<RowVec<T, V>*>(out + (int64_t)t * ld_out)[c] = o;
  }
}

template <typename T, int V>
__global__ __launch_bounds__(64) void k_unpermute_wgrad(const T* __restrict__ dout, int64_t ld_dout,
                                                        const T* __restrict__ rows_, int64_t ld_rows,
                                                        float* __restrict__ dw, const int32_t* __restrict__ inv,
                                                        int tokens, int top_k, int width) {
  const int f = blockIdx.x;  // flat row k * tokens + t
  const int t = f % tokens, k = f / tokens;
  const int j = inv[f];
  if ((unsigned)j >= (unsigned)(tokens * top_k)) {  // (a position outside the table's rows: no row, no gradient)
    if (threadIdx.x == 0) dw[(int64_t)t * top_k + k] = 0.f;
    return;
  }
  const RowVec<T, V>* a = reinterpret_cast<const RowVec<T, V>*>(dout + (int64_t)t * ld_dout);
  const RowVec<T, V>* b = reinterpret_cast<const RowVec<T, V>*>(rows_ + (int64_t)j * ld_rows);
  float acc = 0.f;
  for (int c = threadIdx.x; c < width / V; c += 64) {
    const RowVec<T, V> x = a[c], y = b[c];
#pragma unroll
    for (int i = 0; i < V; ++i) acc += to_f32(x.v[i]) * to_f32(y.v[i]);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) acc += __shfl_xor(acc, d, 64);
  if (threadIdx.x == 0) dw[(int64_t)t * top_k + k] = acc;
}

// whether rows of `width` elements at these strides and addresses can move in 16-byte pieces
template <typename T>
inline bool rows_vectorise(int width, std::initializer_list<int64_t> lds, std::initializer_list<const void*> ptrs) {
  constexpr int V = 16 / (int)sizeof(T);
  if (width % V != 0) return false;
  for (int64_t ld : lds)
    if (ld % V != 0) return false;
  for (const void* p : ptrs)
    if (reinterpret_cast<uintptr_t>(p) & 15u) return false;
  return true;
}

}  // namespace

int launch_segment_build(const void* keys, int key_dtype, int64_t rows, int32_t groups, int64_t* perm_out,
                         int64_t* offsets_out, void* ws, hipStream_t s) {
  SegLayout L(rows, groups);
  SegView V(ws, L);
  const int nblk = (int)L.sort_blocks;
  const int user_groups = groups;
  groups = user_groups + 1;  // the kernels' bucket count: one more for the rows without a group
  const size_t lds = sizeof(int32_t) * (size_t)groups;
  int key_bits = 0;
  while ((1 << key_bits) < groups) ++key_bits;
  if (groups <= kOneGroups && nblk <= kOneBlocks) {
    if (key_dtype == TK_KEY_I32)
      hipLaunchKernelGGL(k_seg_one<int32_t>, dim3(nblk), dim3(kOneWaves * 64), 0, s, (const int32_t*)keys, (int)rows,
                         groups, key_bits, nblk, (int)L.max_tiles, (int)L.max_chunks, (int)L.chunk_tiles, V, perm_out,
                         offsets_out);
    else
      hipLaunchKernelGGL(k_seg_one<int64_t>, dim3(nblk), dim3(kOneWaves * 64), 0, s, (const int64_t*)keys, (int)rows,
                         groups, key_bits, nblk, (int)L.max_tiles, (int)L.max_chunks, (int)L.chunk_tiles, V, perm_out,
                         offsets_out);
    return check_launch();
  }
  if (key_dtype == TK_KEY_I32)
    hipLaunchKernelGGL(k_seg_hist<int32_t>, dim3(nblk), dim3(64), lds, s, (const int32_t*)keys, (int)rows, groups,
                       key_bits, V.hist, V.bad);
  else
    hipLaunchKernelGGL(k_seg_hist<int64_t>, dim3(nblk), dim3(64), lds, s, (const int64_t*)keys, (int)rows, groups,
                       key_bits, V.hist, V.bad);
  hipLaunchKernelGGL(k_seg_scan, dim3(1), dim3(1024), 0, s, (int)rows, groups, nblk, V, (int)L.chunk_tiles,
                     offsets_out);
  // one table entry per thread of the fill blocks (at least one block: an empty input still gets its tables)
  const int fill_blocks = (int)std::min<int64_t>(1024, std::max<int64_t>(1, ceil_div(L.max_tiles, 64)));
  if (key_dtype == TK_KEY_I32)
    hipLaunchKernelGGL(k_seg_scatter<int32_t>, dim3(nblk + fill_blocks), dim3(64), lds, s, (const int32_t*)keys,
                       (int)rows, groups, key_bits, V, perm_out, nblk, (int)L.max_tiles, (int)L.max_chunks,
                       (int)L.chunk_tiles);
  else
    hipLaunchKernelGGL(k_seg_scatter<int64_t>, dim3(nblk + fill_blocks), dim3(64), lds, s, (const int64_t*)keys,
                       (int)rows, groups, key_bits, V, perm_out, nblk, (int)L.max_tiles, (int)L.max_chunks,
                       (int)L.chunk_tiles);
  return check_launch();
}

int launch_class_lists(const int32_t* rank, int n, const RankClass* rc, void* const* lists, int map_rows,
                       const SegView& seg, const SegLayout& L, hipStream_t s) {
  if (n <= 0 || n > kMaxClasses) return TK_ERR_INVALID;
  ClassListArgs p{};
  p.rank = rank;
  p.n = n;
  p.map_rows = map_rows;
  for (int c = 0; c < n; ++c) {
    p.lo[c] = rc[c].lo;
    p.hi[c] = rc[c].hi;
    p.base[c] = (char*)lists[c];
  }
  hipLaunchKernelGGL(k_class_lists, dim3(kNumLists, (unsigned)n), dim3(1024), 0, s, p, ClassListLayout(L), seg,
                     (int)L.max_tiles, (int)L.max_chunks);
  return check_launch();
}

// T = element type; the kernel is instantiated for 16-byte pieces and for single elements
#define TK_ROW_MOVER(KERNEL, T, VEC_OK, GRID, BLOCK, ...)                                    \
  do {                                                                                       \
    if (VEC_OK)                                                                              \
      hipLaunchKernelGGL((KERNEL<T, 16 / (int)sizeof(T)>), GRID, BLOCK, 0, s, __VA_ARGS__);  \
    else                                                                                     \
      hipLaunchKernelGGL((KERNEL<T, 1>), GRID, BLOCK, 0, s, __VA_ARGS__);                    \
  } while (0)

int launch_permute(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, const void* w, const void* ws,
                   int64_t rows, int64_t tokens, int32_t width, int32_t groups, int dtype, hipStream_t s) {
  if (rows == 0) return TK_OK;
  SegLayout L(rows, groups);
  SegView V(ws, L);
  const int top_k = (int)(rows / tokens);
  const dim3 grid((unsigned)ceil_div(L.slots, 4)), block(256);
  if (dtype == TK_DTYPE_F32)
    TK_ROW_MOVER(k_permute, float, rows_vectorise<float>(width, {ld_src, ld_dst}, {src, dst}), grid, block,
                 (const float*)src, ld_src, (float*)dst, ld_dst, (const float*)w, V.slot_row, V.slot_pos, (int)tokens,
                 top_k, width, (int)L.slots);
  else
    TK_ROW_MOVER(k_permute, uint16_t, rows_vectorise<uint16_t>(width, {ld_src, ld_dst}, {src, dst}), grid, block,
                 (const uint16_t*)src, ld_src, (uint16_t*)dst, ld_dst, (const uint16_t*)w, V.slot_row, V.slot_pos,
                 (int)tokens, top_k, width, (int)L.slots);
  return check_launch();
}

int launch_unpermute(const void* rows_, int64_t ld_rows, void* out, int64_t ld_out, const void* w, const void* ws,
                     int64_t rows, int64_t tokens, int32_t width, int32_t groups, int dtype, hipStream_t s) {
  if (tokens == 0) return TK_OK;
  SegLayout L(rows, groups);
  SegView V(ws, L);
  const int top_k = (int)(rows / tokens);
  const dim3 grid((unsigned)tokens), block(256);
  if (dtype == TK_DTYPE_F32)
    TK_ROW_MOVER(k_unpermute, float, rows_vectorise<float>(width, {ld_rows, ld_out}, {rows_, out}), grid, block,
                 (const float*)rows_, ld_rows, (float*)out, ld_out, (const float*)w, V.inv, (int)tokens, top_k, width);
  else
    TK_ROW_MOVER(k_unpermute, uint16_t, rows_vectorise<uint16_t>(width, {ld_rows, ld_out}, {rows_, out}), grid, block,
                 (const uint16_t*)rows_, ld_rows, (uint16_t*)out, ld_out, (const uint16_t*)w, V.inv, (int)tokens, top_k,
                 width);
  return check_launch();
}

int launch_unpermute_wgrad(const void* dout, int64_t ld_dout, const void* rows_, int64_t ld_rows, float* dw,
                           const void* ws, int64_t rows, int64_t tokens, int32_t width, int32_t groups, int dtype,
                           hipStream_t s) {
  if (rows == 0) return TK_OK;
  SegLayout L(rows, groups);
  SegView V(ws, L);
  const int top_k = (int)(rows / tokens);
  const dim3 grid((unsigned)rows), block(64);
  if (dtype == TK_DTYPE_F32)
    TK_ROW_MOVER(k_unpermute_wgrad, float, rows_vectorise<float>(width, {ld_dout, ld_rows}, {dout, rows_}), grid, block,
                 (const float*)dout, ld_dout, (const float*)rows_, ld_rows, dw, V.inv, (int)tokens, top_k, width);
  else
    TK_ROW_MOVER(k_unpermute_wgrad, uint16_t, rows_vectorise<uint16_t>(width, {ld_dout, ld_rows}, {dout, rows_}), grid,
                 block, (const uint16_t*)dout, ld_dout, (const uint16_t*)rows_, ld_rows, dw, V.inv, (int)tokens, top_k,
                 width);
  return check_launch();
}

#undef TK_ROW_MOVER

}  // namespace tk
