// Memory yardsticks: what this GPU sustains for the access patterns of the LoRA kernels, with no arithmetic.
// bench.py --yardstick times them; the kernels of kernels_mfma.hip are judged against these rates as well as
// against the 8 TB/s of the data sheet.  Rows are [rows][width] bf16; `row_of` (optional) is a permutation of
// the rows, taken in tiles of 32 entries like the padded slot table.
#include "tk_mfma.h"

namespace tk {

namespace {

// contiguous streams: 16 B per lane, U accesses in flight per lane
template <int U>
__global__ __launch_bounds__(256) void k_ys_read(const uint4* __restrict__ a, uint4* __restrict__ sink, size_t n) {
  size_t i = (size_t)blockIdx.x * 256 * U + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256 * U;
  uint4 s = zero4();
  for (; i < n; i += stride) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = i + u * 256 < n ? a[i + u * 256] : zero4();
#pragma unroll
    for (int u = 0; u < U; ++u) { s.x ^= v[u].x; s.y ^= v[u].y; s.z ^= v[u].z; s.w ^= v[u].w; }
  }
  if (s.x == 0x12345678u && s.y == 0x9abcdefu) sink[0] = s;  // never true for the fill pattern: keeps the loads
}

__global__ __launch_bounds__(256) void k_ys_copy(const uint4* __restrict__ a, uint4* __restrict__ b, size_t n) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  for (; i < n; i += stride) b[i] = a[i];
}

template <int U, bool NT>
__global__ __launch_bounds__(256) void k_ys_rmw(bf16_t* __restrict__ a, size_t n) {
  size_t i = (size_t)blockIdx.x * 256 * U + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256 * U;
  for (; i < n; i += stride) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (i + u * 256 < n) v[u] = NT ? ld16_nt(a + 8 * (i + u * 256)) : ld16(a + 8 * (i + u * 256));
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (i + u * 256 >= n) continue;
      v[u].x += 0x10001u;
      if (NT) st16_nt(a + 8 * (i + u * 256), v[u]); else st16(a + 8 * (i + u * 256), v[u]);
    }
  }
}

// the expand kernel's pattern: one wave = (tile of 32 rows, 128 columns), a lane holds 8 rows x 16 B, 4 rows x 256 B
// per wave-wide access; read only, or read-modify-write in place with non-temporal accesses
template <bool RMW>
__global__ __launch_bounds__(256) void k_ys_tile(bf16_t* __restrict__ y, const int32_t* __restrict__ row_of, int width,
                                                 int items, uint4* __restrict__ sink) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kb = lane >> 4;
  const int ng = width >> 7;
  const int item = blockIdx.x * 4 + wave;
  if (item >= items) return;
  const int tile = item / ng, c0 = (item - tile * ng) << 7;
  int rows[8];
  if (row_of) {
    const int4 r0 = *reinterpret_cast<const int4*>(row_of + tile * 32 + 4 * kb);
    const int4 r1 = *reinterpret_cast<const int4*>(row_of + tile * 32 + 16 + 4 * kb);
    rows[0] = r0.x; rows[1] = r0.y; rows[2] = r0.z; rows[3] = r0.w;
    rows[4] = r1.x; rows[5] = r1.y; rows[6] = r1.z; rows[7] = r1.w;
  } else {
#pragma unroll
    for (int q = 0; q < 8; ++q) rows[q] = tile * 32 + 16 * (q >> 2) + 4 * kb + (q & 3);
  }
  uint4 v[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    bf16_t* p = y + (int64_t)rows[q] * width + c0 + 8 * li;
    v[q] = RMW ? ld16_nt(p) : ld16(p);
  }
  if (RMW) {
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      v[q].x += 0x10001u;
      st16_nt(y + (int64_t)rows[q] * width + c0 + 8 * li, v[q]);
    }
  } else {
    uint4 s = zero4();
#pragma unroll
    for (int q = 0; q < 8; ++q) { s.x ^= v[q].x; s.y ^= v[q].y; s.z ^= v[q].z; s.w ^= v[q].w; }
    if (s.x == 0x12345678u && s.y == 0x9abcdefu) sink[lane] = s;
  }
}

// the shrink kernel's pattern: one wave = (two tiles, 512 columns), a lane holds 16 B of a row per access, 16 rows x
// 4 pieces of 16 B at a stride of 32 B per wave-wide access, two 64-column steps in flight
__global__ __launch_bounds__(64) void k_ys_shrink(const bf16_t* __restrict__ x, const int32_t* __restrict__ row_of,
                                                  int width, uint4* __restrict__ sink) {
  const int lane = threadIdx.x, li = lane & 15, kb = lane >> 4;
  const int kslices = width >> 9;
  const int pair = blockIdx.x / kslices, ks = blockIdx.x - pair * kslices;
  const bf16_t* r[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int slot = pair * 64 + 16 * q + li;
    r[q] = x + (int64_t)(row_of ? row_of[slot] : slot) * width + 16 * kb + ks * 512;
  }
  uint4 s = zero4();
#pragma unroll
  for (int st = 0; st < 8; st += 2) {
    uint4 v[2][4][2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        v[j][q][0] = ld16(r[q] + (st + j) * 64);
        v[j][q][1] = ld16(r[q] + (st + j) * 64 + 8);
      }
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) { s.x ^= v[j][q][0].x ^ v[j][q][1].y; s.y ^= v[j][q][0].z ^ v[j][q][1].w; }
  }
  if (s.x == 0x12345678u && s.y == 0x9abcdefu) sink[lane] = s;
}

// the row-contraction kernels' pattern: one wave walks a chunk of `chunk_tiles` tiles for 128 columns, two tiles in
// flight (a lane holds 8 rows x 16 B per tile)
__global__ __launch_bounds__(64) void k_ys_walk(const bf16_t* __restrict__ x, const int32_t* __restrict__ row_of,
                                                int width, int chunk_tiles, uint4* __restrict__ sink) {
  const int lane = threadIdx.x, li = lane & 15, kb = lane >> 4;
  const bf16_t* src = x + blockIdx.x * 128 + 8 * li;
  const int tile0 = blockIdx.y * chunk_tiles;
  uint4 s = zero4();
  for (int t = 0; t < chunk_tiles; t += 2) {
    uint4 v[2][8];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      int rows[8];
      const int slot0 = (tile0 + t + u) * 32 + 8 * kb;
      if (row_of) {
        const int4 ra = *reinterpret_cast<const int4*>(row_of + slot0), rb = *reinterpret_cast<const int4*>(row_of + slot0 + 4);
        rows[0] = ra.x; rows[1] = ra.y; rows[2] = ra.z; rows[3] = ra.w; rows[4] = rb.x; rows[5] = rb.y; rows[6] = rb.z; rows[7] = rb.w;
      } else {
#pragma unroll
        for (int q = 0; q < 8; ++q) rows[q] = slot0 + q;
      }
#pragma unroll
      for (int q = 0; q < 8; ++q) v[u][q] = ld16(src + (int64_t)rows[q] * width);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int q = 0; q < 8; ++q) { s.x ^= v[u][q].x; s.y ^= v[u][q].y; s.z ^= v[u][q].z; s.w ^= v[u][q].w; }
  }
  if (s.x == 0x12345678u && s.y == 0x9abcdefu) sink[lane] = s;
}

// the grouped GEMM's operand path: a block of eight waves brings 64 KB per step from global memory straight into
// LDS (eight 16-byte global_load_lds per wave), one step ahead, one barrier per step, and never looks at the data.
// SHARED: every block walks the same 2 MB again and again (every line an L2 hit); else every block walks its own
// contiguous share of the buffer once (every line from memory).
template <bool SHARED>
__global__ __launch_bounds__(512) void k_ys_lds(const char* __restrict__ src, size_t share, int steps,
                                                uint4* __restrict__ sink) {
  __shared__ __attribute__((aligned(1024))) char lds[131072];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const size_t span = SHARED ? ((size_t)2 << 20) : share;  // a multiple of 64 KB (the launcher checks)
  const char* base = SHARED ? src : src + (size_t)blockIdx.x * share;
  for (int s = 0; s < steps; ++s) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const size_t o = ((size_t)s * 65536 + (size_t)(wave * 8 + i) * 1024) % span + lane * 16;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base + o),
                                       (__attribute__((address_space(3))) void*)(lds + (s & 1) * 65536 + (wave * 8 + i) * 1024),
                                       16, 0, 0);
    }
    if (s >= 1) {  // the previous step has landed everywhere before its stage is loaded again
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(0x0070 | 8);  // vmcnt(8) lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
    }
  }
  __syncthreads();
  if (lds[threadIdx.x * 16] == 0x7f && steps < 0) sink[threadIdx.x] = zero4();
}

}  // namespace

}  // namespace tk

using namespace tk;

extern "C" int tk_yardstick(int32_t kind, void* a, void* b, const int32_t* row_of, int64_t rows, int32_t width,
                            tk_stream_t stream) {
  if (!a || !b || rows <= 0 || width <= 0 || rows % 512 != 0 || width % 512 != 0 || rows * width >= (1ll << 40))
    return TK_ERR_INVALID;
  hipStream_t s = (hipStream_t)stream;
  const size_t n16 = (size_t)rows * width / 8;
  bf16_t* x = (bf16_t*)a;
  uint4* sink = (uint4*)b;
  const int tiles = (int)(rows / 32), items = tiles * (width >> 7);
  switch (kind) {
    case TK_YS_READ: hipLaunchKernelGGL(k_ys_read<8>, dim3(4096), dim3(256), 0, s, (const uint4*)a, sink, n16); break;
    case TK_YS_COPY: hipLaunchKernelGGL(k_ys_copy, dim3(4096), dim3(256), 0, s, (const uint4*)a, (uint4*)b, n16); break;
    case TK_YS_RMW: hipLaunchKernelGGL((k_ys_rmw<4, false>), dim3(4096), dim3(256), 0, s, x, n16); break;
    case TK_YS_RMW_NT: hipLaunchKernelGGL((k_ys_rmw<4, true>), dim3(4096), dim3(256), 0, s, x, n16); break;
    case TK_YS_TILE_READ:
      hipLaunchKernelGGL(k_ys_tile<false>, dim3((items + 3) / 4), dim3(256), 0, s, x, row_of, width, items, sink);
      break;
    case TK_YS_TILE_RMW_NT:
      hipLaunchKernelGGL(k_ys_tile<true>, dim3((items + 3) / 4), dim3(256), 0, s, x, row_of, width, items, sink);
      break;
    case TK_YS_SHRINK_READ:
      hipLaunchKernelGGL(k_ys_shrink, dim3((unsigned)(rows / 64 * (width >> 9))), dim3(64), 0, s, x, row_of, width, sink);
      break;
    case TK_YS_WALK_READ:
      hipLaunchKernelGGL(k_ys_walk, dim3(width >> 7, tiles / 16), dim3(64), 0, s, x, row_of, width, 16, sink);
      break;
    case TK_YS_LDS_STREAM:
    case TK_YS_LDS_SHARED: {
      // 256 blocks; a block's share of the buffer in 64 KB steps (TK_YS_LDS_SHARED: sixteen times as many steps)
      const size_t bytes = (size_t)rows * width * 2;
      if (bytes % ((size_t)256 * 65536) != 0 || bytes < ((size_t)2 << 20)) return TK_ERR_INVALID;
      const size_t share = bytes / 256;
      const int steps = (int)(share / 65536);
      if (kind == TK_YS_LDS_STREAM)
        hipLaunchKernelGGL(k_ys_lds<false>, dim3(256), dim3(512), 0, s, (const char*)a, share, steps, sink);
      else
        hipLaunchKernelGGL(k_ys_lds<true>, dim3(256), dim3(512), 0, s, (const char*)a, share, 16 * steps, sink);
      break;
    }
    default: return TK_ERR_INVALID;
  }
  return check_launch();
}
