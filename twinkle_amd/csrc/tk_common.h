// Internal definitions shared by the gfx950 kernels and the C-ABI glue.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

#include "twinkle_amd.h"

namespace tk {

constexpr int kWave = 64;
constexpr int kTileRows = TK_TILE_ROWS;    // rows per forward tile (two 16-row MFMA tiles)
constexpr int kSetTiles = 4;                                    // tiles per work item of the expand above rank 16
constexpr int kRoundFlagBytes = 512;                            // SegView::round_moved: 64 sort blocks x 8 rounds
constexpr int kChunkTilesMin = TK_CHUNK_ROWS / TK_TILE_ROWS;  // smallest weight-gradient chunk: 4 tiles (128 rows)
constexpr int kChunkTilesMax = 128;                             // largest: 4096 rows
constexpr int kSortBlockRows = 512;        // rows one single-wave block orders in the scatter pass

static inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }
static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---------------------------------------------------------------------------
// Device-side segment table.  One allocation, carved by SegLayout from
// (rows, groups) alone, so producer and consumers agree without a host copy.
//
// Kernels work in a *padded* sorted order: every group starts at a multiple of
// 32 slots, so tile i is slots [32 i, 32 i + 32) and a workgroup finds its
// rows from blockIdx with one load (no dependent table walk at kernel start).
// Slots past a group's last row hold -1.
// ---------------------------------------------------------------------------
struct SegHeader {       // 64 x int32, at the start of the workspace
  int32_t magic;
  int32_t rows;
  int32_t groups;
  int32_t num_tiles;     // filled on the device
  int32_t num_chunks;    // filled on the device
  int32_t num_partials;  // chunks that belong to multi-chunk groups
  int32_t bad_keys;      // keys outside [0, groups): rows without a group
  int32_t identity_order;  // 1: the builder left tile_order and set_order as the identity; 0: it computed them, and
                           // SegView::round_moved says whether they differ from the identity
  int32_t pad[56];
};

struct ChunkInfo {  // one weight-gradient chunk: tiles [tile0, tile0 + ntiles) of group `group`, ntiles <= chunk_tiles
  int32_t group;
  int32_t tile0;
  int32_t ntiles;
  int32_t partial;  // slot in the partial buffer, or -1 when the chunk is its group's only one
};

// A chunk is the unit the row contractions (dA, dB) are split into: up to `chunk_tiles` tiles of one
// group.  Every chunk of a multi-chunk group costs one fp32 partial of rank x width, so the chunk
// grows with the batch (about 32 chunks over all rows): the partial traffic stays a fixed small
// fraction of the activations while the number of work items stays in the thousands.  Small batches
// get small chunks: a block walks its chunk tile by tile, one memory latency each, so there the chunk
// length sets the duration of the row-contraction kernels.  A function of the row count alone, so
// producer and consumers agree.
static inline int chunk_tiles_for(int64_t rows) {
  int t = kChunkTilesMin;
  while (t < kChunkTilesMax && (int64_t)t * kTileRows * 32 < rows) t <<= 1;
  return t;
}

// Element (partial slot p, rank index n, column c) of a weight-gradient partial buffer.  Blocks of 128 columns are
// contiguous, [slot][column block][rpad][128]: a launch block leaves its rpad x 128 sums as one run of memory and
// the reduction reads runs of KBs, instead of 512-byte pieces a whole row of the gradient apart.
#ifdef __HIPCC__
#define TK_HD __host__ __device__
#else
#define TK_HD
#endif
TK_HD static inline int64_t partial_slot_floats(int rpad, int width) { return (int64_t)((width + 127) >> 7) * rpad * 128; }
TK_HD static inline int64_t partial_index(int64_t p, int n, int c, int rpad, int width) {
  return (((p * ((width + 127) >> 7) + (c >> 7)) * rpad + n) << 7) + (c & 127);
}

struct SegLayout {
  int64_t rows, groups;
  int64_t sort_blocks;   // ceil(rows / kSortBlockRows)
  int64_t chunk_tiles;   // tiles per weight-gradient chunk (chunk_tiles_for(rows))
  int64_t max_tiles, max_chunks, max_partials;
  int64_t slots;         // padded sorted length: 32 * max_tiles
  // byte offsets from the workspace base
  int64_t off_inv, off_slot_row, off_slot_pos, off_offsets, off_tile_group, off_tile_order, off_set_order, off_round_moved, off_chunks,
      off_tile_first,
      off_chunk_first, off_partial_first, off_hist, off_bad, total;

  SegLayout(int64_t rows_, int64_t groups_) : rows(rows_), groups(groups_) {
    // the builder sorts into groups + 1 buckets: the last one takes the rows whose key is outside
    // [0, groups); its tiles and chunks carry group -1, so no kernel touches those rows
    const int64_t buckets = groups + 1;
    sort_blocks = ceil_div(rows > 0 ? rows : 1, kSortBlockRows);
    max_tiles = ceil_div(rows, kTileRows) + buckets;
    chunk_tiles = chunk_tiles_for(rows);
    max_chunks = ceil_div(rows, chunk_tiles * kTileRows) + buckets;
    max_partials = 2 * ceil_div(rows, chunk_tiles * kTileRows) + 1;
    slots = max_tiles * kTileRows;
    int64_t o = round_up(sizeof(SegHeader), 256);
    off_inv = o;           o += round_up(4 * (rows + 64), 256);
    off_slot_row = o;      o += round_up(4 * slots, 256);
    off_slot_pos = o;      o += round_up(4 * slots, 256);
    off_offsets = o;       o += round_up(4 * (buckets + 1), 256);
    off_tile_group = o;    o += round_up(4 * (max_tiles + 1), 256);
    off_tile_order = o;    o += round_up(4 * (max_tiles + 1), 256);
    off_set_order = o;     o += round_up(4 * (max_tiles / kSetTiles + 2), 256);
    off_round_moved = o;   o += kRoundFlagBytes;
    off_chunks = o;        o += round_up(16 * (max_chunks + 1), 256);
    off_tile_first = o;    o += round_up(4 * (buckets + 1), 256);
    off_chunk_first = o;   o += round_up(4 * (buckets + 1), 256);
    off_partial_first = o; o += round_up(4 * (buckets + 1), 256);
    off_hist = o;          o += round_up(4 * buckets * sort_blocks, 256);
    off_bad = o;           o += round_up(4 * sort_blocks, 256);
    total = o;
  }
};

struct SegView {  // typed device pointers into a segment workspace
  SegHeader* header;
  int32_t* inv;            // [rows]    flat row -> sorted position
  int32_t* slot_row;       // [slots]   padded slot -> flat row (perm), -1 in padding
  int32_t* slot_pos;       // [slots]   padded slot -> sorted position, -1 in padding
  int32_t* offsets;        // [G + 2]  first sorted position of each group; [G] = first row without a group
  int32_t* tile_group;     // [max_tiles]  group of each tile, -1 for rows without a group and past the last tile
  // [max_tiles]  the tiles in the order of their first row ("sweep order"): kernels whose work items are single tiles
  // walk the tiles in this order when rows are reached through slot_row, so that the tiles in flight at any time
  // cover neighbouring rows of the activation tensors whatever their groups (the table is group-major: a group's
  // tiles are spread over all rows).  Identity where the builder does not compute it.
  int32_t* tile_order;
  // [ceil(max_tiles / kSetTiles)]  the same for kernels whose work items are sets of kSetTiles consecutive tiles
  // (tiles kSetTiles s .. kSetTiles s + kSetTiles - 1): the sets in the order of the first row of their first tile
  int32_t* set_order;
  // [64 sort blocks][8 rounds of 64 rows]  one byte per round of the single-launch builder: non-zero when the sort
  // moved a row of the round (its sorted position differs from its row number).  All zero for the rounds of a build
  // <=> the keys came in order <=> tile_order and set_order are the identity.  Bytes of rounds past the last row of
  // the current build are stale.
  uint8_t* round_moved;
  ChunkInfo* chunks;       // [max_chunks]
  int32_t* tile_first;     // [G + 2]  first tile of each group
  int32_t* chunk_first;    // [G + 2]  first chunk of each group
  int32_t* partial_first;  // [G + 2]  first partial slot of each multi-chunk group
  int32_t* hist;           // [sort_blocks][G + 1]  per-block histogram, then per-block exclusive bases
  int32_t* bad;            // [sort_blocks]  out-of-range keys seen by each block
  SegView(const void* base, const SegLayout& L) {
    char* b = (char*)base;
    header = (SegHeader*)b;
    inv = (int32_t*)(b + L.off_inv);
    slot_row = (int32_t*)(b + L.off_slot_row);
    slot_pos = (int32_t*)(b + L.off_slot_pos);
    offsets = (int32_t*)(b + L.off_offsets);
    tile_group = (int32_t*)(b + L.off_tile_group);
    tile_order = (int32_t*)(b + L.off_tile_order);
    set_order = (int32_t*)(b + L.off_set_order);
    round_moved = (uint8_t*)(b + L.off_round_moved);
    chunks = (ChunkInfo*)(b + L.off_chunks);
    tile_first = (int32_t*)(b + L.off_tile_first);
    chunk_first = (int32_t*)(b + L.off_chunk_first);
    partial_first = (int32_t*)(b + L.off_partial_first);
    hist = (int32_t*)(b + L.off_hist);
    bad = (int32_t*)(b + L.off_bad);
  }
  // rows of the activation tensors, by padded slot
  const int32_t* slot_table(int map_rows) const { return map_rows ? slot_row : slot_pos; }
  // order in which single-tile work items take the tiles (null: as numbered; rows in segment order are contiguous)
  const int32_t* tile_walk(int map_rows) const { return map_rows ? tile_order : nullptr; }
  const int32_t* set_walk(int map_rows) const { return map_rows ? set_order : nullptr; }
};

constexpr int32_t kSegMagic = 0x544b5347;  // "TKSG"

// ---------------------------------------------------------------------------
// Saved shrink output, indexed by padded slot.  hT[n][slot]: rank index major,
// so the row-contraction kernels read 8 consecutive slots per lane; followed
// by hrow[slot][n], the expand kernel's operand.
// ---------------------------------------------------------------------------
static inline int64_t h_ld(int64_t rows, int64_t groups) { return round_up(SegLayout(rows, groups).slots, 64); }
// Padded rank: 16, 32, 64 or 128 (the kernels are instantiated per padded rank).
static inline int32_t rank_pad(int32_t max_rank) {
  int32_t p = 16;
  while (p < max_rank) p <<= 1;
  return p;
}
static inline int elt_bytes(int dtype) { return dtype == TK_DTYPE_BF16 ? 2 : 4; }

// Rank classes (tk_lora_desc::rank_classes).  A launch serves the groups whose rank lies in (lo, hi]: hi is the
// launch's padded rank, lo the padded rank of the class below (0 for the lowest class or when there is one class
// only).  Every kernel turns a group's rank into its live rank with this: 0 (skip) outside the window.
TK_HD static inline int class_rank(int r, int lo, int hi) { return (r > lo && r <= hi) ? r : 0; }
constexpr int kMaxClasses = 4;
struct RankClass {
  int32_t lo, hi;  // ranks lo < r <= hi; hi is the max_rank of the class's descriptor
};
// The classes of a descriptor, lowest first; one class (0, max_rank] unless the caller listed several.
static inline int rank_classes_of(const tk_lora_desc& d, RankClass (&out)[kMaxClasses]) {
  static const int32_t bound[kMaxClasses + 1] = {0, 16, 32, 64, 128};
  int n = 0;
  const int m = d.rank_classes & ((1 << kMaxClasses) - 1);
  if ((m & (m - 1)) != 0) {  // more than one bit
    // a class's window starts where the listed class below it ends, so a rank between two listed classes is served
    // by the upper one (a mask can be too coarse, never lose a group)
    for (int c = 0; c < kMaxClasses; ++c)
      if (((m >> c) & 1) && bound[c] < d.max_rank) {
        const int32_t lo = n ? out[n - 1].hi : 0;
        out[n++] = RankClass{lo, std::min(bound[c + 1], d.max_rank)};
      }
  }
  if (n <= 1) {
    out[0] = RankClass{0, d.max_rank};
    n = 1;
  }
  return n;
}

// The MFMA shrink kernel covers the source width with blocks of shrink_waves() waves, each wave
// taking kShrinkSteps steps of 64 columns; wider sources are split over several blocks whose
// partial sums meet in a global buffer.
constexpr int kShrinkSteps = 8;
static inline int shrink_waves(int rpad) { return rpad <= 16 ? 1 : (rpad <= 32 ? 2 : 4); }
static inline int shrink_kslices(int width, int rpad) {
  return (int)ceil_div(ceil_div(width, 64), (int64_t)kShrinkSteps * shrink_waves(rpad));
}
// Above rank 16, with long groups and a source of 1024 to 4096 columns, the shrink runs as k_shrink_quad: blocks of
// (eight tiles, `steps` steps of 64 columns).  The slices are cut so that all blocks are resident at once where
// the row count allows (two blocks of four waves per CU, 256 CUs): a launch of 1.02 rounds costs two.  Wider
// sources stay with k_shrink_pair (measured at 14336 columns, rank 64: 304 us against 236; there a block's short
// look-ahead along each of its 256 rows costs more than the shared weights save).
constexpr int kQuadResident = 512;
struct ShrinkPlan {
  int kslices;     // slices per tile
  int quad_steps;  // 0: k_shrink_pair; else steps per slice of k_shrink_quad
};
static inline ShrinkPlan shrink_plan(int64_t rows, int64_t groups, int width, int rpad) {
  const int nsteps = (int)ceil_div(width, 64);
  if (rpad <= 16 || nsteps < 16 || nsteps > 64 || rows < 8 * kTileRows * groups)
    return ShrinkPlan{shrink_kslices(width, rpad), 0};
  const int64_t sets = ceil_div(rows, 8 * kTileRows);
  int ks = (int)std::min<int64_t>(kQuadResident / sets, nsteps / 8);
  ks = std::max(ks, 2);
  const int steps = (int)ceil_div(nsteps, ks);
  return ShrinkPlan{(int)ceil_div(nsteps, steps), steps};  // no empty slice at the end
}
static inline int64_t shrink_partial_bytes(int64_t rows, int64_t groups, int width, int rpad) {
  const int ks = std::max(shrink_kslices(width, rpad), shrink_plan(rows, groups, width, rpad).kslices);
  return ks > 1 ? round_up(SegLayout(rows, groups).max_tiles * ks * (int64_t)kTileRows * rpad * 4, 256) : 0;
}

// The single-pass backward kernel (padded rank 16 or 32, width a multiple of 512) leaves one slice of dh per
// 512 columns, which at rank 32 is twice the slices of the shrink kernel it replaces.
static inline int fused_dy_kslices(int width, int rpad) {
  return ((rpad == 16 || rpad == 32) && width % 512 == 0 && width >= 1024) ? width / 512 : 0;
}
static inline int64_t bwd_partial_bytes(int64_t rows, int64_t groups, int width, int rpad) {
  const int ks = std::max(std::max(shrink_kslices(width, rpad), shrink_plan(rows, groups, width, rpad).kslices),
                          fused_dy_kslices(width, rpad));
  return ks > 1 ? round_up(SegLayout(rows, groups).max_tiles * ks * (int64_t)kTileRows * rpad * 4, 256) : 0;
}

// bf16 copies of fp32 adapter weights (tk_lora_desc::weights_f32): pointer tables [G] for A and B, then
// A_g as [rpad][in_features] and B_g as [out_features][rpad] for every group.
struct WeightStage {
  int64_t off_ptr_a, off_ptr_b, off_a, off_b, total;
  int64_t stride_a, stride_b;  // elements per group
  WeightStage() : off_ptr_a(0), off_ptr_b(0), off_a(0), off_b(0), total(0), stride_a(0), stride_b(0) {}
  WeightStage(int64_t groups, int64_t rpad, int64_t in_features, int64_t out_features) {
    stride_a = rpad * in_features;
    stride_b = out_features * rpad;
    int64_t o = 0;
    off_ptr_a = o;  o += round_up(8 * groups, 256);
    off_ptr_b = o;  o += round_up(8 * groups, 256);
    off_a = o;      o += round_up(2 * groups * stride_a, 256);
    off_b = o;      o += round_up(2 * groups * stride_b, 256);
    total = o;
  }
};
static inline bool mixed_weights(const tk_lora_desc& d) { return d.weights_f32 != 0 && d.dtype == TK_DTYPE_BF16; }
static inline int64_t weight_stage_bytes(const tk_lora_desc& d) {
  return mixed_weights(d) ? WeightStage(d.num_groups, rank_pad(d.max_rank), d.in_features, d.out_features).total : 0;
}

// Backward workspace carving.
struct BwdLayout {
  int64_t off_dh, off_hpart, off_wT_shrink, off_wT_expand, off_part_a, off_part_b, total;
  int64_t rpad, ldh;
  BwdLayout(const tk_lora_desc& d) {
    SegLayout S(d.rows, d.num_groups);
    rpad = rank_pad(d.max_rank);
    ldh = h_ld(d.rows, d.num_groups);
    const int64_t e = elt_bytes(d.dtype);
    int64_t o = 0;
    off_dh = o;         o += round_up(2 * rpad * ldh * e, 256);  // rank-major + slot-major copies
    off_hpart = o;      o += bwd_partial_bytes(d.rows, d.num_groups, d.out_features, (int)rpad);
    // B^T per group [rpad][M]  (shrink weight of the backward pass)
    off_wT_shrink = o;  o += round_up((int64_t)d.num_groups * rpad * d.out_features * e, 256);
    // A^T per group [K][rpad]  (expand weight of the backward pass)
    off_wT_expand = o;  o += round_up((int64_t)d.num_groups * rpad * d.in_features * e, 256);
    off_part_a = o;     o += round_up(S.max_partials * rpad * round_up(d.in_features, 128) * 4, 256);
    off_part_b = o;     o += round_up(S.max_partials * rpad * round_up(d.out_features, 128) * 4, 256);
    total = o;
  }
};

// What a consumer of a segment table may index with: every group number, row number, tile range and partial slot that a
// kernel reads from the table (caller-held memory) is compared with these before it is used as an index, and an entry
// outside them is treated as absent (no group, no row, an empty chunk).  A table that was overwritten or belongs to
// another batch then gives wrong results for the tiles concerned, not accesses outside the caller's tensors.
struct TableBounds {
  int32_t groups;        // group numbers are in [0, groups)
  int32_t rows;          // row numbers (slot_row / slot_pos entries) are in [0, rows)
  int32_t max_tiles;     // tile numbers are in [0, max_tiles)
  int32_t chunk_tiles;   // a chunk has at most this many tiles
  int32_t max_partials;  // partial slots are in [0, max_partials)
  int32_t max_chunks;    // chunk numbers are in [0, max_chunks)
};
static inline TableBounds table_bounds(const SegLayout& L) {
  return TableBounds{(int32_t)L.groups, (int32_t)L.rows, (int32_t)L.max_tiles, (int32_t)L.chunk_tiles,
                     (int32_t)L.max_partials, (int32_t)L.max_chunks};
}

// Work list of a launch that serves one rank class out of several: the ids of the work items (tiles, pairs of tiles,
// chunks ..) that hold a group of the class, and their number, both on the device (built per call by
// launch_class_lists from the segment table and the ranks).  The grid still covers every item of the table; blocks
// past *count leave at once, and the live ones are dense at the front.  ids == nullptr: items are taken as numbered.
struct WorkList {
  const int32_t* ids;
  const int32_t* count;
};
enum { kListTiles = 0, kListPairs = 1, kListOcts = 2, kListSets = 3, kListChunks = 4, kNumLists = 5 };
// One class's lists inside a caller-provided buffer: counts[8], then the five id arrays.
struct ClassListLayout {
  int64_t off[kNumLists], items[kNumLists], total;
  explicit ClassListLayout(const SegLayout& L) {
    items[kListTiles] = L.max_tiles;                          // tiles, in sweep order when rows are gathered
    items[kListPairs] = ceil_div(L.max_tiles, 2);             // tiles 2 p, 2 p + 1
    items[kListOcts] = ceil_div(L.max_tiles, 8);              // tiles 8 o .. 8 o + 7
    items[kListSets] = ceil_div(L.max_tiles, kSetTiles);      // tiles 4 s .. 4 s + 3, in set order when rows are gathered
    items[kListChunks] = L.max_chunks;
    int64_t o = 256;                                          // counts
    for (int i = 0; i < kNumLists; ++i) {
      off[i] = o;
      o += round_up(4 * (items[i] + 1), 256);
    }
    total = o;
  }
  WorkList list(const void* base, int which) const {
    return WorkList{(const int32_t*)((const char*)base + off[which]), (const int32_t*)base + which};
  }
};
static inline int64_t class_list_bytes(int64_t rows, int64_t groups) { return ClassListLayout(SegLayout(rows, groups)).total; }

// Everything one pass of the (shrink, expand) pair needs.  The forward pass
// and the input-gradient pass are the same computation with the roles of the
// weights swapped, so both are described by this one struct.
struct PassArgs {
  const void* src;   int64_t ld_src;   // rows that are shrunk     (x  | dy)
  void* dst;         int64_t ld_dst;   // rows that are updated    (y  | dx), may be null
  void* hT;          int64_t ldh;      // shrink output            (h  | dh), written
  // shrink weight of group g: rank-major [r][width_src]
  const void* const* w_shrink;  const void* w_shrink_base;  int64_t ld_shrink;  int64_t shrink_group_stride;
  // expand weight of group g: column-major-by-output [width_dst][r]
  const void* const* w_expand;  const void* w_expand_base;  int64_t ld_expand;  int64_t expand_group_stride;
  const int32_t* rank;
  const float* scale;
  int32_t width_src;  // K | M
  int32_t width_dst;  // M | K
  int32_t map_rows;
  int32_t rpad;
  int32_t src_rows;  // rows of src / dst (bound for speculative row addresses)
  float* hpart;          // partial sums of the split shrink, [tile][slice][32][rpad]
  int32_t kslices;       // blocks per tile of the MFMA shrink
  int32_t quad_steps;    // 0: k_shrink_pair; else k_shrink_quad with this many 64-column steps per slice
  // the expand weight's rows are permuted inside every group of 128 (TransposeJob::swizzle_a): the row of
  // column c0 + 8 i + q lies at c0 + 16 q + i, so that the 16 rows one MFMA operand load touches are adjacent
  int32_t expand_swizzled;
  // groups whose rank is not in (rank_lo, rpad] are skipped (see class_rank); class_mode != 0 says that such groups
  // may exist, and kernels then look at the rank before they request a tile's rows
  int32_t rank_lo, class_mode;
  WorkList wl_tiles, wl_pairs, wl_octs, wl_sets;  // class_mode: the items of this class (see WorkList)
  TableBounds tb;
};

// Optional side job of a weight-gradient launch (bf16 MFMA path): the first `y_blocks` rows of the
// grid write the transposed weight copies the input-gradient pass reads, bT_g[n][m] = B_g[m][n] and
// aT_g[k][n] = A_g[n][k] (zero for n >= rank[g]), instead of spending a launch of their own on them.
struct TransposeJob {
  const void* const* lora_A;  int64_t lda;
  const void* const* lora_B;  int64_t ldb;
  void* aT;  // [groups][in_features][rpad]
  void* bT;  // [groups][rpad][out_features]
  int32_t in_features, out_features, groups;
  int32_t y_blocks;  // 0: no job
  int32_t swizzle_a; // aT rows permuted inside every 128 (see PassArgs::expand_swizzled); in_features % 128 == 0
  int32_t skip_dead; // leave entries at and beyond a group's rank unwritten (the MFMA kernels never read them)
  int32_t src_f32;   // lora_A / lora_B hold fp32 (lda, ldb in fp32 elements); the copies are bf16 all the same
  int32_t rank_lo;   // groups of rank <= rank_lo (or above the padded rank) are skipped
};

// Row-contraction (weight gradient) pass: out_g[n][c] = sum_p hT[n][p] * src[row(p)][c].
struct WgradArgs {
  const void* src;  int64_t ld_src;   // x | dy
  const void* hT;   int64_t ldh;      // dh | h
  float* partial;                     // [max_partials][width / 128][rpad][128], see partial_index
  void* const* grad;                  // device array [G]
  int64_t ld_grad;
  const int32_t* rank;
  int32_t width;       // K | M
  int32_t transposed;  // 0: grad_g is [r][width] (dA); 1: grad_g is [width][r] (dB)
  int32_t accumulate;
  int32_t map_rows;
  int32_t rpad;
  int32_t grad_f32;    // the gradients (and the adapter weights a kernel reads next to them) are fp32 whatever the
                       // element type of src (tk_lora_desc::weights_f32)
  int32_t rank_lo;     // groups whose rank is not in (rank_lo, rpad] are skipped (see class_rank)
  int32_t pair_chunks; // the launch takes two consecutive chunks of a group as one work item (see chunk_follows)
  WorkList wl_chunks;  // several rank classes: the chunks of this class
  TableBounds tb;
  TransposeJob tr;
};

// Projections that share their input (kernels_shared.hip).
constexpr int kMaxShared = 4;
struct SharedShrinkArgs {
  const void* src;  int64_t ld_src;      // x
  int32_t width_src, src_rows, map_rows, kslices, nproj;
  const void* const* w[kMaxShared];      // device pointer tables [G] of A_p, rank-major [r][K]
  int64_t ld_w[kMaxShared];
  const int32_t* rank[kMaxShared];       // device [G]
  float* hpart[kMaxShared];              // split-shrink buffer of projection p, [tile][slice][32][16]
  TableBounds tb;
};
struct SharedExpandArgs {
  void* dst;  int64_t ld_dst;            // dx
  int32_t width_dst, map_rows, nproj;
  const void* hrow[kMaxShared];          // slot-major dh of projection p, [slots][rpad]
  const void* aT[kMaxShared];            // A_p^T copies, [G][K][rpad]
  const int32_t* rank[kMaxShared];
  TableBounds tb;
};
struct SharedWgradArgs {                 // dA_p for all p from one pass over x (w[p].src / ld_src / width agree)
  int32_t nproj;
  WgradArgs w[kMaxShared];
};
struct PassJobs {
  PassArgs p[kMaxShared];
};
struct DyFusedJob {
  WgradArgs a;                  // dB job of one projection (src = dy_p); a.tr carries the weight transposes
  const void* const* lora_B;    // device pointer table [G] of B_p
  int64_t ldb;
  float* hpart;                 // split-shrink buffer receiving the slices of dh_p
  int32_t kslices, x_blocks;    // x_blocks is filled in by the launcher
};
struct DyFusedJobs {
  DyFusedJob j[kMaxShared];
  int32_t n;
  int32_t x_first[kMaxShared + 1];  // job p owns the blocks x_first[p] <= blockIdx.x < x_first[p + 1]
};
struct WgradReduceJobs {
  int32_t n;
  WgradArgs a[2 * kMaxShared];
};
// bf16 copies of the fp32 weights of `d` (layout: WeightStage at `stage`), with their pointer tables
int launch_convert_weights(const tk_lora_desc& d, void* stage, bool want_a, bool want_b, hipStream_t s);
// the same for up to kMaxShared descriptors (projections that share their input) in one launch
int launch_convert_weights_multi(const tk_lora_desc* const* d, void* const* stage, int n, bool want_a, bool want_b,
                                 hipStream_t s);
int launch_transpose_job(const TransposeJob& t, const int32_t* rank, int rpad, hipStream_t s);
int launch_dy_fused_multi(const DyFusedJob* jobs, int n, const SegView& seg, const SegLayout& L, hipStream_t s);
int launch_pass_multi(const PassArgs* a, int n, const SegView& seg, const SegLayout& L, int phases, hipStream_t s);
int launch_wgrad_reduce_multi(const WgradArgs* sets, int n, const SegView& seg, const SegLayout& L, hipStream_t s);
int launch_shrink_shared(const SharedShrinkArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s);
int launch_expand_shared(const SharedExpandArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s);
int launch_wgrad_shared(const SharedWgradArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s);
// projections of one padded rank 32 or 64 that share their input
int launch_shrink_multi(const PassArgs* a, int n, const SegView& seg, const SegLayout& L, hipStream_t s);
int launch_expand_shared_wide(const SharedExpandArgs& a, int rpad, const SegView& seg, const SegLayout& L, hipStream_t s);
int launch_wgrad_coop_multi(const SharedWgradArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s);

// kernels_grouped.hip
struct GroupedPlanEntry {  // a row block of the grouped GEMM: up to 4 consecutive tiles of one expert
  int32_t tile0, ntiles, expert;
  int32_t first, count;  // the expert's row blocks are the entries [first, first + count)
  int32_t pad;
};
struct GroupedArgs {
  const uint16_t* x;  int64_t ldx;                     // activations, rows reached through the slot table
  const uint16_t* w;  int64_t w_stride, ldw;           // packed weights: expert e at w + e * w_stride, [N][K]
  int32_t w_rows_are_inputs;                           // ... or [K][N]: y = x W (no LoRA term then)
  uint16_t* y;        int64_t ldy;
  int32_t K, N, src_rows, map_rows;
  // LoRA term (rpad = 0: none): y += h B_g^T with h[slot][rpad] as the shrink kernels leave it
  const void* const* lora_B;  int64_t ldb;
  const int32_t* rank;  int32_t rpad;
  const uint16_t* hrow;
  TableBounds tb;
};
bool grouped_gemm_supported(const GroupedArgs& a);
int64_t grouped_plan_entries(const SegLayout& L, int64_t experts);
int launch_grouped_gemm(const GroupedArgs& a, int experts, int nt, GroupedPlanEntry* plan, int32_t* nblocks,
                        const SegView& seg, const SegLayout& L, hipStream_t s);

// kernels_act.hip: out = silu(gate) * up (dout null) or its backward into out = d(gate | up)
int launch_swiglu(const void* gate_up, int64_t ld_in, const void* dout, int64_t ld_dout, void* out, int64_t ld_out,
                  int64_t rows, int inter, int dtype, hipStream_t s);

// kernels_segments.hip
// work lists of `n` rank classes (ranks in (lo[c], hi[c]]) into lists[c] (ClassListLayout each)
int launch_class_lists(const int32_t* rank, int n, const RankClass* rc, void* const* lists, int map_rows,
                       const SegView& seg, const SegLayout& L, hipStream_t s);
int launch_segment_build(const void* keys, int key_dtype, int64_t rows, int32_t groups, int64_t* perm_out,
                         int64_t* offsets_out, void* ws, hipStream_t s);
int launch_permute(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, const void* w, const void* ws,
                   int64_t rows, int64_t tokens, int32_t width, int32_t groups, int dtype, hipStream_t s);
int launch_unpermute(const void* rows_, int64_t ld_rows, void* out, int64_t ld_out, const void* w, const void* ws,
                     int64_t rows, int64_t tokens, int32_t width, int32_t groups, int dtype, hipStream_t s);
int launch_unpermute_wgrad(const void* dout, int64_t ld_dout, const void* rows_, int64_t ld_rows, float* dw,
                           const void* ws, int64_t rows, int64_t tokens, int32_t width, int32_t groups, int dtype,
                           hipStream_t s);

// kernels_generic.hip : any shape / stride, fp32 and bf16, VALU
int launch_pass_generic(const PassArgs& a, const SegView& seg, const SegLayout& L, int dtype, int phases,
                        hipStream_t s);
int launch_wgrad_generic(const WgradArgs& a, const SegView& seg, const SegLayout& L, int dtype, hipStream_t s);
// sums the chunk partials of up to two contractions (dA, dB; either may be null) in one launch
int launch_wgrad_reduce(const WgradArgs* a0, const WgradArgs* a1, const SegView& seg, const SegLayout& L, int dtype,
                        hipStream_t s);
int launch_transpose_weights(const tk_lora_desc& d, int rank_lo, void* bT, void* aT, hipStream_t s);

// kernels_optim.hip : multi-tenant gradient norm and AdamW
int launch_opt_grad_norm(const tk_opt_tensor* tensors, int n_tensors, const tk_opt_tenant* tenants, int n_tenants,
                         int64_t max_numel, int dtype, float* norm_out, float* clip_out, float* partial, hipStream_t s);
int launch_opt_adamw(const tk_opt_tensor* tensors, int n_tensors, const tk_opt_tenant* tenants, int64_t max_numel,
                     int dtype, const float* clip, int flags, hipStream_t s);
int64_t opt_partial_floats(int n_tensors, int64_t max_numel);

// kernels_mfma.hip : bf16, aligned shapes, MFMA
bool pass_mfma_supported(const PassArgs& a);
// `phases` (bit mask): 1 = shrink, 2 = expand (h already written), 4 = only the last step of a split shrink
// (its slices are already in a.hpart)
int launch_pass_mfma(const PassArgs& a, const SegView& seg, const SegLayout& L, int phases, hipStream_t s);
bool wgrad_mfma_supported(const WgradArgs& a);
// a.tr.y_blocks is chosen by the launcher when a.tr.aT is set
int launch_wgrad_mfma(const WgradArgs& a, const SegView& seg, const SegLayout& L, hipStream_t s);
// dB and the slices of the dy shrink from one pass over dy (a: the dB contraction; a.tr may carry the aT copy)
bool dy_fused_supported(const WgradArgs& a, int kslices);
int launch_dy_fused(const WgradArgs& a, const void* const* lora_B, int64_t ldb, float* hpart, int kslices,
                    const SegView& seg, const SegLayout& L, hipStream_t s);

}  // namespace tk
