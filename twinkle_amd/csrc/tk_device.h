// Device-side helpers shared by the kernel translation units.
#pragma once

#include "tk_common.h"

namespace tk {

typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ inline float to_f32(float v) { return v; }
__device__ inline float to_f32(bf16_t v) { return __uint_as_float((uint32_t)v << 16); }

__device__ inline bf16_t f32_to_bf16(float v) {
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40);  // NaN stays NaN
  u += 0x7fffu + ((u >> 16) & 1u);                                         // round to nearest even
  return (bf16_t)(u >> 16);
}
__device__ inline void from_f32(float v, float* o) { *o = v; }
__device__ inline void from_f32(float v, bf16_t* o) { *o = f32_to_bf16(v); }

// Weight of group g: either a per-group pointer (caller-owned slot tensors)
// or base + g * stride (a packed copy inside a workspace).
template <typename T>
__device__ inline const T* group_weight(const void* const* ptrs, const void* base, int64_t stride, int g) {
  return ptrs ? (const T*)ptrs[g] : (const T*)base + (int64_t)g * stride;
}

// Entries of the segment table before they are used as indices (see TableBounds).
__device__ inline int checked_group(int g, const TableBounds& tb) { return (unsigned)g < (unsigned)tb.groups ? g : -1; }
__device__ inline int checked_row(int r, const TableBounds& tb) { return (unsigned)r < (unsigned)tb.rows ? r : -1; }
__device__ inline int checked_tile(int t, const TableBounds& tb) { return (unsigned)t < (unsigned)tb.max_tiles ? t : -1; }
// a chunk whose tile range or partial slot lies outside the table counts as a chunk of no group
__device__ inline ChunkInfo checked_chunk(ChunkInfo ci, const TableBounds& tb) {
  const bool ok = ci.tile0 >= 0 && ci.ntiles >= 0 && ci.ntiles <= tb.chunk_tiles && ci.tile0 <= tb.max_tiles - ci.ntiles &&
                  ci.partial < tb.max_partials;
  ci.group = ok ? checked_group(ci.group, tb) : -1;
  return ci;
}

// Weight-gradient launches at padded rank 64 take two consecutive chunks of a group as one work item
// (WgradArgs::pair_chunks): their partial sums are 64 x width floats per chunk, written once and read once by the
// reduction, and half as many of them are worth more there than the parallelism of short chunks (config 5's q
// projection: 40 partials of 1 MB per gradient).  Chunk `b` is taken by the block of the chunk `a` in front of it
// when both belong to one group, b's partial slot is odd and the two are neighbours in slots and in tiles; the
// block of `b` then has nothing to do and the reduction leaves b's slot out (see live_partial).  Both blocks
// evaluate this on the same two checked entries.
__device__ inline bool chunk_follows(const ChunkInfo& a, const ChunkInfo& b) {
  return b.group >= 0 && a.group == b.group && (b.partial & 1) && a.partial == b.partial - 1 &&
         b.tile0 == a.tile0 + a.ntiles;
}
// The m-th partial slot (counted from the group's first, `pf`) that holds a sum when chunks are paired, and how
// many of a group's `nchunk` slots do: the first always, after it the even slots.
__device__ inline int live_partial(int m, int pf) { return m == 0 ? 0 : 2 * m - (pf & 1); }
__device__ inline int live_partials(int nchunk, int pf) { return 1 + ((pf & 1) ? nchunk / 2 : (nchunk - 1) / 2); }

// Work item i of a launch: the i-th id of the launch's work list, -1 past its end (see WorkList); i itself without one.
__device__ inline int work_item(const WorkList& wl, int i) {
  if (!wl.ids) return i;
  return i < *wl.count ? wl.ids[i] : -1;
}

inline int check_launch() { return hipGetLastError() == hipSuccess ? TK_OK : TK_ERR_LAUNCH; }

}  // namespace tk
