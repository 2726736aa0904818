// C ABI of the library: argument checks, workspace carving, kernel choice.
#include <stdlib.h>

#include <mutex>
#include <vector>

#include "tk_common.h"

using namespace tk;

namespace {

// a list of several rank classes must be a list of classes and contain the class of max_rank (every layout is sized
// from the listed classes)
bool classes_ok(const tk_lora_desc* d) {
  const int m = d->rank_classes;
  if (m < 0 || m >= (1 << kMaxClasses)) return false;
  if ((m & (m - 1)) == 0) return true;  // none or one: one class, padded to max_rank
  const int top = d->max_rank <= 16 ? 0 : d->max_rank <= 32 ? 1 : d->max_rank <= 64 ? 2 : 3;
  return ((m >> top) & 1) != 0 && (m >> (top + 1)) == 0;
}

bool desc_ok(const tk_lora_desc* d) {
  if (!d) return false;
  if (d->rows < 0 || d->rows >= (1ll << 31)) return false;
  if (d->in_features <= 0 || d->out_features <= 0) return false;
  if (d->num_groups <= 0 || d->num_groups > TK_MAX_GROUPS) return false;
  if (d->max_rank < 0 || d->max_rank > TK_MAX_RANK) return false;
  if (d->dtype != TK_DTYPE_F32 && d->dtype != TK_DTYPE_BF16) return false;
  if (!d->seg_ws || !d->lora_A || !d->lora_B || !d->rank || !d->scale) return false;
  if (d->lda < d->in_features || d->ldb < d->max_rank) return false;
  if (d->weights_f32 != 0 && (d->weights_f32 != 1 || d->dtype != TK_DTYPE_BF16)) return false;
  if (!classes_ok(d)) return false;
  return true;
}

// fp32 adapter weights next to bf16 activations: the kernels read bf16 copies made at `stage` (layout: WeightStage).
// The descriptor the kernels work from once the copies exist: the copies' pointer tables and strides (gradients keep
// the caller's strides, see bwd).
void staged_desc(const tk_lora_desc* d, void* stage, tk_lora_desc* out) {
  const int rpad = rank_pad(d->max_rank);
  const WeightStage W(d->num_groups, rpad, d->in_features, d->out_features);
  *out = *d;
  out->weights_f32 = 0;
  out->lora_A = (const void* const*)((char*)stage + W.off_ptr_a);
  out->lora_B = (const void* const*)((char*)stage + W.off_ptr_b);
  out->lda = d->in_features;
  out->ldb = rpad;
}

// makes the copies and returns that descriptor
int stage_weights(const tk_lora_desc* d, void* stage, bool want_a, bool want_b, hipStream_t s, tk_lora_desc* out) {
  const int rc = launch_convert_weights(*d, stage, want_a, want_b, s);
  if (rc != TK_OK) return rc;
  staged_desc(d, stage, out);
  return TK_OK;
}

// TK_FORCE_GENERIC=1 in the environment routes every launch to the shape-agnostic kernels
// (an A/B switch for debugging; both families are HIP kernels on the GPU).
bool force_generic() {
  static const bool v = [] {
    const char* e = getenv("TK_FORCE_GENERIC");
    return e && e[0] == '1';
  }();
  return v;
}

// The backward pass has two independent chains that meet only at the end (dB needs dy and h; dX and
// dA need the dy shrink), and no single kernel of either reaches the memory system's peak, so the
// library runs them on two streams: the caller's and one of its own per device (default priority,
// non-blocking), forked and joined with events.  TK_BWD_STREAMS=0 keeps everything on the caller's stream.
struct SideStream {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, mid = nullptr, join = nullptr;
  int state = 0;  // 0: not created yet, 1: ready, -1: creation failed (single-stream fallback)
  std::mutex use;  // held while a call enqueues its fork .. join sequence: the events are shared per device
};

SideStream* side_stream() {
  static const bool enabled = [] {
    const char* e = getenv("TK_BWD_STREAMS");
    return !(e && e[0] == '0');
  }();
  if (!enabled) return nullptr;
  constexpr int kMaxDevices = 64;
  static SideStream side[kMaxDevices];
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  SideStream& x = side[dev];
  if (x.state == 0) {
    const bool ok = hipStreamCreateWithFlags(&x.stream, hipStreamNonBlocking) == hipSuccess &&
                    hipEventCreateWithFlags(&x.fork, hipEventDisableTiming) == hipSuccess &&
                    hipEventCreateWithFlags(&x.mid, hipEventDisableTiming) == hipSuccess &&
                    hipEventCreateWithFlags(&x.join, hipEventDisableTiming) == hipSuccess;
    x.state = ok ? 1 : -1;
    if (!ok) (void)hipGetLastError();
  }
  return x.state == 1 ? &x : nullptr;
}

// Several rank classes in one call (tk_lora_desc::rank_classes) are independent chains of launches over disjoint
// rows and groups, and no single kernel reaches the memory system's peak, so the classes above the first run on
// streams of the library's own (per device, default priority, non-blocking), forked from and joined to the caller's
// stream with events: the start-up and the tail of one class's launches are covered by the others' work.
// TK_CLASS_STREAMS=0 keeps every class on the caller's stream.
struct ClassStreams {
  hipStream_t stream[kMaxClasses - 1] = {};
  hipEvent_t fork = nullptr, join[kMaxClasses - 1] = {};
  int state = 0;   // 0: not created yet, 1: ready, -1: creation failed (single-stream fallback)
  std::mutex use;  // held while a call enqueues its fork .. join sequence: the events are shared per device
};

ClassStreams* class_streams() {
  static const bool enabled = [] {
    const char* e = getenv("TK_CLASS_STREAMS");
    return !(e && e[0] == '0');
  }();
  if (!enabled) return nullptr;
  constexpr int kMaxDevices = 64;
  static ClassStreams cs[kMaxDevices];
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  ClassStreams& x = cs[dev];
  if (x.state == 0) {
    bool ok = hipEventCreateWithFlags(&x.fork, hipEventDisableTiming) == hipSuccess;
    for (int i = 0; ok && i < kMaxClasses - 1; ++i)
      ok = hipStreamCreateWithFlags(&x.stream[i], hipStreamNonBlocking) == hipSuccess &&
           hipEventCreateWithFlags(&x.join[i], hipEventDisableTiming) == hipSuccess;
    x.state = ok ? 1 : -1;
    if (!ok) (void)hipGetLastError();
  }
  return x.state == 1 ? &x : nullptr;
}

// Runs body(c, stream, forked) for every class: the highest class on the caller's stream (forked = false), the others
// on the library's class streams between a fork and a join (forked = true), or all on the caller's stream where
// there are none.  Everything
// enqueued on `s` before the call is visible to every class; everything every class enqueued is complete for what
// follows on `s`.  A body that is told `forked` must not fork again: a fork inside a forked stream is more than the
// runtime's stream capture takes (it crashed when such a capture was ended), and the classes already overlap.
template <typename Body>
int for_each_class(int n, hipStream_t s, Body body) {
  ClassStreams* cs = n > 1 ? class_streams() : nullptr;
  if (!cs) {
    for (int c = 0; c < n; ++c) {
      const int rc = body(c, s, false);
      if (rc != TK_OK) return rc;
    }
    return TK_OK;
  }
  std::lock_guard<std::mutex> guard(cs->use);
  if (hipEventRecord(cs->fork, s) != hipSuccess) return TK_ERR_LAUNCH;
  for (int c = 0; c + 1 < n; ++c)
    if (hipStreamWaitEvent(cs->stream[c], cs->fork, 0) != hipSuccess) return TK_ERR_LAUNCH;
  // once forked, every stream joins again, also after an error: none may be left attached to the caller's stream
  // (or to a graph capture of it)
  int rc = TK_OK;
  for (int c = 0; c + 1 < n; ++c) {  // the library's streams first: they start while the caller's is being filled
    const int r = body(c, cs->stream[c], true);
    if (r != TK_OK && rc == TK_OK) rc = r;
  }
  {
    // The highest class stays on the caller's stream, where it may fork once more: it is the one with the longest
    // chain of kernels (above rank 32 dy is read by two of them, which then run side by side).
    const int r = body(n - 1, s, false);
    if (r != TK_OK && rc == TK_OK) rc = r;
  }
  for (int c = 0; c + 1 < n; ++c)
    if (hipEventRecord(cs->join[c], cs->stream[c]) != hipSuccess ||
        hipStreamWaitEvent(s, cs->join[c], 0) != hipSuccess)
      return TK_ERR_LAUNCH;
  return rc;
}

// Scratch of tk_lora_fwd_noalloc: the shrink output h and the partial sums of a split shrink, which tk_lora_fwd takes
// from the caller.  One copy per GPU, held until the process ends.  The name below is a host-side stand-in, not a
// device address: host code only ever uses the address that hipGetSymbolAddress returns for the current device.
static __device__ __align__(256) unsigned char scratch[TK_NOALLOC_SCRATCH_BYTES];

// Device address of `scratch` on the current device, looked up once per device.
int scratch_address(void** out) {
  constexpr int kMaxDevices = 64;
  static void* ptr[kMaxDevices];
  static bool known[kMaxDevices];
  static std::mutex mu;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return TK_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(mu);
  if (!known[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
      (void)hipGetLastError();
      return TK_ERR_LAUNCH;
    }
    ptr[dev] = p;
    known[dev] = true;
  }
  *out = ptr[dev];
  return TK_OK;
}

int run_pass(const PassArgs& a, const SegView& V, const SegLayout& L, int dtype, int phases, hipStream_t s) {
  if (dtype == TK_DTYPE_BF16 && !force_generic() && pass_mfma_supported(a))
    return launch_pass_mfma(a, V, L, phases, s);
  return launch_pass_generic(a, V, L, dtype, phases, s);
}

int run_wgrad(const WgradArgs& a, const SegView& V, const SegLayout& L, int dtype, hipStream_t s) {
  int rc;
  if (dtype == TK_DTYPE_BF16 && !force_generic() && wgrad_mfma_supported(a))
    rc = launch_wgrad_mfma(a, V, L, s);
  else
    rc = launch_wgrad_generic(a, V, L, dtype, s);
  return rc;
}

}  // namespace

extern "C" {

const char* tk_version(void) { return "twinkle_amd 0.1 (gfx950)"; }

const char* tk_error_string(int code) {
  switch (code) {
    case TK_OK: return "ok";
    case TK_ERR_INVALID: return "invalid argument";
    case TK_ERR_WORKSPACE: return "workspace too small";
    case TK_ERR_UNSUPPORTED: return "unsupported shape";
    case TK_ERR_LAUNCH: return "HIP launch error";
    case TK_ERR_SCRATCH: return "problem too large for the library's built-in scratch buffer";
    default: return "unknown error";
  }
}

int64_t tk_segment_workspace_bytes(int64_t rows, int32_t num_groups) {
  if (rows < 0 || num_groups <= 0) return TK_ERR_INVALID;
  return SegLayout(rows, num_groups).total;
}

int tk_segment_build(const void* keys, int32_t key_dtype, int64_t rows, int32_t num_groups, int64_t* perm_out,
                     int64_t* offsets_out, void* seg_ws, int64_t seg_ws_bytes, tk_stream_t stream) {
  if (rows < 0 || num_groups <= 0 || !seg_ws || (rows > 0 && !keys)) return TK_ERR_INVALID;
  if (key_dtype != TK_KEY_I32 && key_dtype != TK_KEY_I64) return TK_ERR_INVALID;
  if (num_groups > TK_MAX_GROUPS || rows >= (1ll << 31)) return TK_ERR_UNSUPPORTED;
  if (seg_ws_bytes < SegLayout(rows, num_groups).total) return TK_ERR_WORKSPACE;
  return launch_segment_build(keys, key_dtype, rows, num_groups, perm_out, offsets_out, seg_ws,
                              (hipStream_t)stream);
}

int tk_segment_bad_keys(const void* seg_ws, tk_stream_t stream, int64_t* count_out) {
  if (!seg_ws || !count_out) return TK_ERR_INVALID;
  SegHeader h;
  if (hipMemcpyAsync(&h, seg_ws, sizeof(h), hipMemcpyDeviceToHost, (hipStream_t)stream) != hipSuccess)
    return TK_ERR_LAUNCH;
  if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) return TK_ERR_LAUNCH;
  if (h.magic != kSegMagic) return TK_ERR_INVALID;
  *count_out = h.bad_keys;
  return TK_OK;
}

// Host-side check of a segment table: the whole workspace is copied back and every array is rebuilt from the
// group sizes and the row order it holds, entry by entry.
int tk_segment_validate(const void* seg_ws, int64_t rows, int32_t num_groups, tk_stream_t stream,
                        int32_t* failed_check_out, int64_t* index_out) {
  if (!seg_ws || rows < 0 || rows >= (1ll << 31) || num_groups <= 0 || num_groups > TK_MAX_GROUPS) return TK_ERR_INVALID;
  const SegLayout L(rows, num_groups);
  std::vector<char> host((size_t)L.total);
  if (hipMemcpyAsync(host.data(), seg_ws, (size_t)L.total, hipMemcpyDeviceToHost, (hipStream_t)stream) != hipSuccess)
    return TK_ERR_LAUNCH;
  if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) return TK_ERR_LAUNCH;
  const SegView V(host.data(), L);
  const int G = num_groups, B = G + 1;  // buckets: the groups, then the rows without a group
  auto fail = [&](int check, int64_t index) {
    if (failed_check_out) *failed_check_out = check;
    if (index_out) *index_out = index;
    return TK_ERR_INVALID;
  };
  if (failed_check_out) *failed_check_out = 0;
  if (index_out) *index_out = -1;
  const SegHeader& h = *V.header;
  // 1: header
  if (h.magic != kSegMagic || h.rows != rows || h.groups != G || h.num_tiles < 0 || h.num_tiles > L.max_tiles ||
      h.num_chunks < 0 || h.num_chunks > L.max_chunks || h.num_partials < 0 || h.num_partials > L.max_partials ||
      h.bad_keys < 0 || h.bad_keys > rows)
    return fail(1, 0);
  // 2: offsets
  if (V.offsets[0] != 0 || V.offsets[B] != rows || V.offsets[G] != rows - h.bad_keys) return fail(2, 0);
  for (int g = 0; g < B; ++g)
    if (V.offsets[g + 1] < V.offsets[g]) return fail(2, g);
  // 3: first tile of every bucket
  if (V.tile_first[0] != 0 || V.tile_first[B] != h.num_tiles) return fail(3, 0);
  for (int g = 0; g < B; ++g)
    if (V.tile_first[g + 1] - V.tile_first[g] != ceil_div(V.offsets[g + 1] - V.offsets[g], kTileRows)) return fail(3, g);
  // 4: group of every tile; 5: rows and positions of every slot; 7: rows ascending inside a group
  std::vector<int32_t> seen((size_t)rows, 0);
  for (int g = 0; g < B; ++g) {
    int32_t prev = -1;
    for (int t = V.tile_first[g]; t < V.tile_first[g + 1]; ++t) {
      if (V.tile_group[t] != (g < G ? g : -1)) return fail(4, t);
      for (int i = 0; i < kTileRows; ++i) {
        const int64_t s_ = (int64_t)t * kTileRows + i;
        const int64_t pos = V.offsets[g] + (int64_t)(t - V.tile_first[g]) * kTileRows + i;
        const int32_t row = V.slot_row[s_];
        if (pos >= V.offsets[g + 1]) {
          if (row != -1 || V.slot_pos[s_] != -1) return fail(5, s_);
          continue;
        }
        if (V.slot_pos[s_] != pos || row < 0 || row >= rows) return fail(5, s_);
        if (seen[row]++) return fail(6, s_);          // 6: every row exactly once
        if (V.inv[row] != pos) return fail(6, row);   //    and inv is the inverse
        if (row <= prev) return fail(7, s_);          // 7: stable order
        prev = row;
      }
    }
  }
  for (int64_t t = h.num_tiles; t < L.max_tiles; ++t) {
    if (V.tile_group[t] != -1) return fail(4, t);
    for (int i = 0; i < kTileRows; ++i)
      if (V.slot_row[t * kTileRows + i] != -1 || V.slot_pos[t * kTileRows + i] != -1) return fail(5, t * kTileRows + i);
  }
  for (int64_t r = 0; r < rows; ++r)
    if (!seen[r]) return fail(6, r);
  // 8: the walk orders are permutations of the tiles / of the sets of four tiles
  {
    std::vector<char> hit((size_t)L.max_tiles, 0);
    for (int64_t i = 0; i < L.max_tiles; ++i) {
      const int32_t t = V.tile_order[i];
      if (t < 0 || t >= L.max_tiles || hit[t]++) return fail(8, i);
    }
    const int64_t sets = ceil_div(L.max_tiles, kSetTiles);
    std::vector<char> hit_s((size_t)sets, 0);
    for (int64_t i = 0; i < sets; ++i) {
      const int32_t t = V.set_order[i];
      if (t < 0 || t >= sets || hit_s[t]++) return fail(8, L.max_tiles + i);
    }
  }
  // 9: chunks; 10: first chunk and first partial slot of every bucket
  int32_t chunk = 0, partial = 0;
  for (int g = 0; g < B; ++g) {
    if (V.chunk_first[g] != chunk) return fail(10, g);
    const int ntile = V.tile_first[g + 1] - V.tile_first[g];
    const int nchunk = (int)ceil_div(ntile, L.chunk_tiles);
    const bool multi = nchunk > 1 && g < G;
    if (V.partial_first[g] != partial) return fail(10, g);
    for (int j = 0; j < nchunk; ++j, ++chunk) {
      if (chunk >= L.max_chunks) return fail(9, chunk);
      const ChunkInfo& c = V.chunks[chunk];
      if (c.group != (g < G ? g : -1) || c.tile0 != V.tile_first[g] + j * (int)L.chunk_tiles ||
          c.ntiles != std::min<int>((int)L.chunk_tiles, ntile - j * (int)L.chunk_tiles) ||
          c.partial != (multi ? partial + j : -1))
        return fail(9, chunk);
    }
    if (multi) partial += nchunk;
  }
  if (V.chunk_first[B] != chunk || chunk != h.num_chunks || V.partial_first[B] != partial || partial != h.num_partials ||
      partial > L.max_partials)
    return fail(10, B);
  for (int64_t c = chunk; c < L.max_chunks; ++c)
    if (V.chunks[c].group != -1) return fail(9, c);
  return TK_OK;
}

static bool rows_args_ok(const void* a, const void* b, const void* ws, int64_t rows, int64_t tokens, int32_t width,
                         int32_t groups, int32_t dtype) {
  if (!ws || rows < 0 || tokens < 0 || width <= 0 || groups <= 0) return false;
  if (rows > 0 && (!a || !b || tokens == 0 || rows % tokens != 0)) return false;
  return dtype == TK_DTYPE_F32 || dtype == TK_DTYPE_BF16;
}

int tk_permute_rows(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, const void* weights,
                    const void* seg_ws, int64_t rows, int64_t num_tokens, int32_t width, int32_t num_groups,
                    int32_t dtype, tk_stream_t stream) {
  if (!rows_args_ok(src, dst, seg_ws, rows, num_tokens, width, num_groups, dtype)) return TK_ERR_INVALID;
  if (ld_src < width || ld_dst < width) return TK_ERR_INVALID;
  return launch_permute(src, ld_src, dst, ld_dst, weights, seg_ws, rows, num_tokens, width, num_groups, dtype,
                        (hipStream_t)stream);
}

int tk_unpermute_rows(const void* rows_p, int64_t ld_rows, void* out, int64_t ld_out, const void* weights,
                      const void* seg_ws, int64_t rows, int64_t num_tokens, int32_t width, int32_t num_groups,
                      int32_t dtype, tk_stream_t stream) {
  if (!rows_args_ok(rows_p, out, seg_ws, rows, num_tokens, width, num_groups, dtype)) return TK_ERR_INVALID;
  if (ld_rows < width || ld_out < width) return TK_ERR_INVALID;
  return launch_unpermute(rows_p, ld_rows, out, ld_out, weights, seg_ws, rows, num_tokens, width, num_groups, dtype,
                          (hipStream_t)stream);
}

int tk_unpermute_weight_grad(const void* dout, int64_t ld_dout, const void* rows_p, int64_t ld_rows, float* dw,
                             const void* seg_ws, int64_t rows, int64_t num_tokens, int32_t width,
                             int32_t num_groups, int32_t dtype, tk_stream_t stream) {
  if (!rows_args_ok(dout, rows_p, seg_ws, rows, num_tokens, width, num_groups, dtype) || (rows > 0 && !dw))
    return TK_ERR_INVALID;
  if (ld_dout < width || ld_rows < width) return TK_ERR_INVALID;
  return launch_unpermute_wgrad(dout, ld_dout, rows_p, ld_rows, dw, seg_ws, rows, num_tokens, width, num_groups,
                                dtype, (hipStream_t)stream);
}

// what the size queries need of a descriptor: shapes and dtype, no pointers
static bool desc_shape_ok(const tk_lora_desc* d) {
  return d && d->rows >= 0 && d->num_groups > 0 && d->num_groups <= TK_MAX_GROUPS && d->max_rank >= 0 &&
         d->max_rank <= TK_MAX_RANK && d->in_features > 0 && d->out_features > 0 &&
         (d->dtype == TK_DTYPE_F32 || d->dtype == TK_DTYPE_BF16) &&
         (d->weights_f32 == 0 || (d->weights_f32 == 1 && d->dtype == TK_DTYPE_BF16)) && classes_ok(d);
}

// h without the staged weight copies that follow it when the adapters are fp32
static int64_t h_core_bytes(const tk_lora_desc* d) {
  const int rpad = rank_pad(d->max_rank);
  return round_up(2 * (int64_t)rpad * h_ld(d->rows, d->num_groups) * elt_bytes(d->dtype), 256) +
         shrink_partial_bytes(d->rows, d->num_groups, d->in_features, rpad);
}

// The rank classes of a backward call (tk_lora_desc::rank_classes): for each class the descriptor its launches work
// from (max_rank = the top of the class, so every workspace layout takes the class's padded rank) and where its region
// of the workspace starts.  One class, equal to the caller's descriptor, unless several were listed.  The forward
// pass is not split: all groups run on the kernels of the largest padded rank there (a launch per class costs the
// in-place update of y more than the narrower kernels save; measured on 32 adapters of ranks 8 .. 64, 4096 -> 14336:
// 539 against 472 us), so h has one layout, and every class of the backward reads its groups' rows of it.
struct ClassPlan {
  int n;
  RankClass rc[kMaxClasses];
  tk_lora_desc d[kMaxClasses];
  int64_t ws_off[kMaxClasses], ws_bytes[kMaxClasses];
  int64_t ws_core_total;
  // several classes: their work lists (ClassListLayout each) follow the classes' regions; every call rebuilds them
  int64_t list_bytes, ws_total;
  void* lists[kMaxClasses];  // filled in by build_lists
};

static ClassPlan class_plan(const tk_lora_desc* d) {
  ClassPlan P{};
  P.n = rank_classes_of(*d, P.rc);
  for (int c = 0; c < P.n; ++c) {
    P.d[c] = *d;
    P.d[c].max_rank = P.rc[c].hi;
    P.ws_off[c] = P.ws_core_total;
    P.ws_bytes[c] = BwdLayout(P.d[c]).total;
    P.ws_core_total += P.ws_bytes[c];
  }
  P.list_bytes = P.n > 1 ? class_list_bytes(d->rows, d->num_groups) : 0;
  P.ws_total = P.ws_core_total + P.n * P.list_bytes;
  return P;
}

// Several classes: builds their work lists at `base` (see ClassPlan) and hands them to a pass / a contraction.
static int build_lists(ClassPlan& P, const tk_lora_desc* d, void* base, const SegView& V, const SegLayout& L,
                       hipStream_t s) {
  if (P.n <= 1) return TK_OK;
  for (int c = 0; c < P.n; ++c) P.lists[c] = (char*)base + c * P.list_bytes;
  return launch_class_lists(d->rank, P.n, P.rc, P.lists, d->map_rows, V, L, s);
}
static void use_lists(const ClassPlan& P, int c, const SegLayout& L, PassArgs* a, WgradArgs* ga, WgradArgs* gb) {
  if (P.n <= 1) return;
  const ClassListLayout CL(L);
  if (a) {
    a->wl_tiles = CL.list(P.lists[c], kListTiles);
    a->wl_pairs = CL.list(P.lists[c], kListPairs);
    a->wl_octs = CL.list(P.lists[c], kListOcts);
    a->wl_sets = CL.list(P.lists[c], kListSets);
  }
  if (ga) ga->wl_chunks = CL.list(P.lists[c], kListChunks);
  if (gb) gb->wl_chunks = CL.list(P.lists[c], kListChunks);
}

int64_t tk_lora_h_bytes(const tk_lora_desc* d) {
  if (!desc_shape_ok(d)) return TK_ERR_INVALID;
  // rank-major copy hT[rpad][ld], slot-major copy hrow[ld][rpad], then the partial sums of a split shrink, then
  // the bf16 copies of fp32 adapter weights
  return h_core_bytes(d) + weight_stage_bytes(*d);
}

int64_t tk_lora_bwd_workspace_bytes(const tk_lora_desc* d) {
  if (!desc_shape_ok(d)) return TK_ERR_INVALID;
  return class_plan(d).ws_total;
}

// Arguments of the forward pass h = scale x A^T, y += h B^T.  Null x / y are replaced by placeholders: shapes are
// checked against what both phases need, so that the two halves of one forward pick the same kernels.
static PassArgs fwd_pass_args(const tk_lora_desc* d, const void* x, int64_t ldx, void* y, int64_t ldy, void* h,
                              int rank_lo = 0, int class_mode = 0) {
  PassArgs a{};
  a.rank_lo = rank_lo;  a.class_mode = class_mode;
  a.tb = table_bounds(SegLayout(d->rows, d->num_groups));
  a.src = x ? x : h;  a.ld_src = x ? ldx : d->in_features;
  a.dst = y ? y : h;  a.ld_dst = y ? ldy : d->out_features;
  a.hT = h;   a.ldh = h_ld(d->rows, d->num_groups);
  a.w_shrink = d->lora_A;  a.ld_shrink = d->lda;
  a.w_expand = d->lora_B;  a.ld_expand = d->ldb;
  a.rank = d->rank;  a.scale = d->scale;
  a.width_src = d->in_features;  a.width_dst = d->out_features;
  a.map_rows = d->map_rows;  a.rpad = rank_pad(d->max_rank);  a.src_rows = (int32_t)d->rows;
  a.hpart = (float*)((char*)h + round_up(2 * (int64_t)a.rpad * a.ldh * elt_bytes(d->dtype), 256));
  const ShrinkPlan plan = shrink_plan(d->rows, d->num_groups, d->in_features, a.rpad);
  a.kslices = plan.kslices;  a.quad_steps = plan.quad_steps;
  return a;
}

// Everything the backward of one projection needs, carved from its workspace.
struct BwdPlan {
  WgradArgs ga{}, gb{};  // dA[n][k] = sum_rows dh[row][n] x[row][k];  dB[m][n] = sum_rows dy[row][m] h[row][n]
  PassArgs a{};          // dh = scale * dy B, dx += dh A
  TransposeJob tr{};     // B^T, A^T copies
  void* dh = nullptr;
  void* bT = nullptr;
  void* aT = nullptr;
};

static BwdPlan bwd_plan(const tk_lora_desc* d, const BwdLayout& B, const void* dy, int64_t lddy, const void* x,
                        int64_t ldx, const void* h, void* dx, int64_t lddx, void* const* grad_A, void* const* grad_B,
                        int32_t accumulate, void* ws, int rank_lo = 0, int class_mode = 0) {
  BwdPlan p;
  p.ga.rank_lo = p.gb.rank_lo = p.a.rank_lo = p.tr.rank_lo = rank_lo;
  p.a.class_mode = class_mode;
  p.ga.tb = p.gb.tb = p.a.tb = table_bounds(SegLayout(d->rows, d->num_groups));
  char* w = (char*)ws;
  p.dh = w + B.off_dh;
  p.bT = w + B.off_wT_shrink;
  p.aT = w + B.off_wT_expand;
  if (grad_B) {
    WgradArgs& g = p.gb;
    g.src = dy;  g.ld_src = lddy;
    g.hT = h;    g.ldh = B.ldh;
    g.partial = (float*)(w + B.off_part_b);
    g.grad = grad_B;  g.ld_grad = d->ldb;
    g.rank = d->rank;  g.width = d->out_features;  g.transposed = 1;
    g.accumulate = accumulate;  g.map_rows = d->map_rows;  g.rpad = (int32_t)B.rpad;
  }
  if (grad_A) {
    WgradArgs& g = p.ga;
    g.src = x;  g.ld_src = ldx;
    g.hT = p.dh;  g.ldh = B.ldh;
    g.partial = (float*)(w + B.off_part_a);
    g.grad = grad_A;  g.ld_grad = d->lda;
    g.rank = d->rank;  g.width = d->in_features;  g.transposed = 0;
    g.accumulate = accumulate;  g.map_rows = d->map_rows;  g.rpad = (int32_t)B.rpad;
  }
  PassArgs& a = p.a;
  a.src = dy;  a.ld_src = lddy;
  a.dst = dx;  a.ld_dst = lddx;
  a.hT = p.dh;   a.ldh = B.ldh;
  a.w_shrink_base = p.bT;  a.ld_shrink = d->out_features;  a.shrink_group_stride = B.rpad * d->out_features;
  a.w_expand_base = p.aT;  a.ld_expand = B.rpad;           a.expand_group_stride = B.rpad * d->in_features;
  a.rank = d->rank;  a.scale = d->scale;
  a.width_src = d->out_features;  a.width_dst = d->in_features;
  a.map_rows = d->map_rows;  a.rpad = (int32_t)B.rpad;  a.src_rows = (int32_t)d->rows;
  a.hpart = (float*)(w + B.off_hpart);
  const ShrinkPlan plan = shrink_plan(d->rows, d->num_groups, d->out_features, a.rpad);
  a.kslices = plan.kslices;  a.quad_steps = plan.quad_steps;
  TransposeJob& tr = p.tr;
  tr.lora_A = d->lora_A;  tr.lda = d->lda;
  tr.lora_B = d->lora_B;  tr.ldb = d->ldb;
  tr.aT = p.aT;  tr.bT = p.bT;
  tr.in_features = d->in_features;  tr.out_features = d->out_features;  tr.groups = d->num_groups;
  // fp32 adapters under bf16 activations: the backward kernels read the weights only through the transposed
  // copies (made from the fp32 matrices directly) and, in the fused pass over dy, B itself; the gradients are fp32
  tr.src_f32 = p.ga.grad_f32 = p.gb.grad_f32 = mixed_weights(*d) ? 1 : 0;
  // padded rank 64 on the two-wave MFMA kernel (the test run_wgrad makes): chunks are taken in pairs
  const bool coop = d->dtype == TK_DTYPE_BF16 && !force_generic() && B.rpad == 64;
  p.ga.pair_chunks = coop && grad_A && wgrad_mfma_supported(p.ga);
  p.gb.pair_chunks = coop && grad_B && wgrad_mfma_supported(p.gb);
  return p;
}

static int lora_pass_fwd(const tk_lora_desc* d, const void* x, int64_t ldx, void* y, int64_t ldy, void* h,
                         int phases, tk_stream_t stream) {
  if (!desc_ok(d) || !h) return TK_ERR_INVALID;
  if (d->rows == 0 || d->max_rank == 0) return TK_OK;
  if ((phases & 1) && (!x || ldx < d->in_features)) return TK_ERR_INVALID;
  if ((phases & 2) && (!y || ldy < d->out_features)) return TK_ERR_INVALID;
  SegLayout L(d->rows, d->num_groups);
  SegView V(d->seg_ws, L);
  tk_lora_desc staged;
  if (mixed_weights(*d)) {  // each half of the forward converts the matrix it reads
    const int rc = stage_weights(d, (char*)h + h_core_bytes(d), (phases & 1) != 0, (phases & 2) != 0,
                                 (hipStream_t)stream, &staged);
    if (rc != TK_OK) return rc;
    d = &staged;
  }
  const PassArgs a = fwd_pass_args(d, x, ldx, y, ldy, h);
  return run_pass(a, V, L, d->dtype, phases, (hipStream_t)stream);
}

int tk_lora_fwd(const tk_lora_desc* d, const void* x, int64_t ldx, void* y, int64_t ldy, void* h,
                tk_stream_t stream) {
  return lora_pass_fwd(d, x, ldx, y, ldy, h, 3, stream);
}

int tk_lora_fwd_noalloc(const tk_lora_desc* d, const void* x, int64_t ldx, void* y, int64_t ldy, tk_stream_t stream) {
  if (!desc_ok(d)) return TK_ERR_INVALID;
  const int64_t need = tk_lora_h_bytes(d);
  if (need < 0) return (int)need;
  if (need > (int64_t)TK_NOALLOC_SCRATCH_BYTES) return TK_ERR_SCRATCH;
  if (d->rows == 0 || d->max_rank == 0) return TK_OK;
  void* h = nullptr;
  const int rc = scratch_address(&h);
  if (rc != TK_OK) return rc;
  // nothing in h has to start at zero: every entry a live tile reads is written by this call first
  return lora_pass_fwd(d, x, ldx, y, ldy, h, 3, stream);
}

int tk_lora_shrink(const tk_lora_desc* d, const void* x, int64_t ldx, void* h, tk_stream_t stream) {
  return lora_pass_fwd(d, x, ldx, nullptr, 0, h, 1, stream);
}

int tk_lora_expand(const tk_lora_desc* d, const void* h, void* y, int64_t ldy, tk_stream_t stream) {
  return lora_pass_fwd(d, nullptr, 0, y, ldy, const_cast<void*>(h), 2, stream);
}

// The backward of the groups of one rank class (d: the class's descriptor; every group when there is one class).
static int lora_bwd_class(const tk_lora_desc* d, const ClassPlan& P, int c, const void* dy, int64_t lddy,
                          const void* x, int64_t ldx, const void* h, void* dx, int64_t lddx, void* const* grad_A,
                          void* const* grad_B, int32_t accumulate, void* ws, hipStream_t s, bool may_fork) {
  const int rank_lo = P.rc[c].lo, class_mode = P.n > 1;
  BwdLayout B(*d);
  SegLayout L(d->rows, d->num_groups);
  SegView V(d->seg_ws, L);
  int rc;
  const bool need_wT = dx || grad_A;
  BwdPlan plan = bwd_plan(d, B, dy, lddy, x, ldx, h, dx, lddx, grad_A, grad_B, accumulate, ws, rank_lo, class_mode);
  use_lists(P, c, L, &plan.a, &plan.ga, &plan.gb);
  WgradArgs &ga = plan.ga, &gb = plan.gb;
  PassArgs& a = plan.a;
  const TransposeJob& tr = plan.tr;
  void *bT = plan.bT, *aT = plan.aT;
  const bool mfma = d->dtype == TK_DTYPE_BF16 && !force_generic();

  const int fused_ks = fused_dy_kslices(d->out_features, a.rpad);
  if (grad_B && need_wT && mfma && pass_mfma_supported(a) && fused_ks && dy_fused_supported(gb, fused_ks)) {
    // One pass over dy yields dB and the slices of dh (and, on the side, the A^T copy for dX).
    a.kslices = fused_ks;
    gb.tr = tr;
    gb.tr.bT = nullptr;
    // written here, read only by the expand below (the flat kernel of padded rank 16 wants its rows permuted)
    gb.tr.swizzle_a = a.expand_swizzled = (a.rpad == 16);
    rc = launch_dy_fused(gb, d->lora_B, d->ldb, a.hpart, a.kslices, V, L, s);
    gb.tr = TransposeJob{};
    if (rc != TK_OK) return rc;
    if ((rc = launch_pass_mfma(a, V, L, dx ? 4 | 2 : 4, s)) != TK_OK) return rc;
    if (grad_A && (rc = run_wgrad(ga, V, L, d->dtype, s)) != TK_OK) return rc;
    return launch_wgrad_reduce(grad_A ? &ga : nullptr, &gb, V, L, d->dtype, s);
  }

  // Separate kernels.  Two chains that meet only at the end: dB (reads dy and h) runs on a side stream,
  // the dy shrink -> dX on the caller's; dA follows the shrink on the side stream, next to the expand.
  // Without a side stream everything runs in the same order on the caller's stream.
  SideStream* side = (grad_B && need_wT && may_fork) ? side_stream() : nullptr;
  hipStream_t s2 = side ? side->stream : s;
  // two host threads must not interleave their records and waits on the device's one set of events
  std::unique_lock<std::mutex> side_guard;
  if (side) side_guard = std::unique_lock<std::mutex>(side->use);
  if (side) {
    if (hipEventRecord(side->fork, s) != hipSuccess || hipStreamWaitEvent(s2, side->fork, 0) != hipSuccess)
      return TK_ERR_LAUNCH;
  }
  // once forked, every path joins again, also after an error: the side stream must not be left attached to
  // the caller's stream (or to a graph capture of it)
  rc = TK_OK;
  do {
    bool wT_done = false;
    if (grad_B) {
      if (!side && need_wT && mfma && wgrad_mfma_supported(gb) && d->out_features % 8 == 0) {
        gb.tr = tr;  // one stream: the MFMA launch also writes the transposed weight copies of the pass below
        wT_done = true;
      }
      rc = run_wgrad(gb, V, L, d->dtype, s2);
      gb.tr = TransposeJob{};
      if (rc != TK_OK) break;
    }
    if (need_wT) {
      if (!wT_done) {
        // both consumers on the MFMA kernels: 16-byte stores, dead rank indices skipped; else the generic copy
        const bool fast = mfma && pass_mfma_supported(a) && d->out_features % 8 == 0;
        rc = fast ? launch_transpose_job(tr, d->rank, a.rpad, s) : launch_transpose_weights(*d, rank_lo, bT, aT, s);
        if (rc != TK_OK) break;
      }
      if ((rc = run_pass(a, V, L, d->dtype, 1, s)) != TK_OK) break;
      if (side && grad_A) {  // dh is complete: the side stream may start dA while dX runs here
        if (hipEventRecord(side->mid, s) != hipSuccess || hipStreamWaitEvent(s2, side->mid, 0) != hipSuccess) {
          rc = TK_ERR_LAUNCH;
          break;
        }
      }
      if (dx && (rc = run_pass(a, V, L, d->dtype, 2, s)) != TK_OK) break;
    }
    if (grad_A && (rc = run_wgrad(ga, V, L, d->dtype, s2)) != TK_OK) break;
    // the chunk partials of both contractions are summed by one launch
    rc = launch_wgrad_reduce(grad_A ? &ga : nullptr, grad_B ? &gb : nullptr, V, L, d->dtype, s2);
  } while (false);
  if (side) {
    if (hipEventRecord(side->join, s2) != hipSuccess || hipStreamWaitEvent(s, side->join, 0) != hipSuccess)
      return TK_ERR_LAUNCH;
  }
  return rc;
}

int tk_lora_bwd(const tk_lora_desc* d, const void* dy, int64_t lddy, const void* x, int64_t ldx, const void* h,
                void* dx, int64_t lddx, void* const* grad_A, void* const* grad_B, int32_t accumulate, void* ws,
                int64_t ws_bytes, tk_stream_t stream) {
  if (!desc_ok(d)) return TK_ERR_INVALID;
  if (d->rows == 0 || d->max_rank == 0) return TK_OK;
  if (!dy || lddy < d->out_features || !ws) return TK_ERR_INVALID;
  if (dx && lddx < d->in_features) return TK_ERR_INVALID;
  if (grad_A && (!x || ldx < d->in_features)) return TK_ERR_INVALID;
  if (grad_B && !h) return TK_ERR_INVALID;
  ClassPlan P = class_plan(d);
  if (ws_bytes < P.ws_total) return TK_ERR_WORKSPACE;
  {
    SegLayout L(d->rows, d->num_groups);
    SegView V(d->seg_ws, L);
    const int rc = build_lists(P, d, (char*)ws + P.ws_core_total, V, L, (hipStream_t)stream);
    if (rc != TK_OK) return rc;
  }
  // Every rank class reads and writes the rows and the gradients of its own groups only, in its own region of the
  // workspace; of h (one layout, written by the forward at the largest padded rank) it reads the rank-major copy,
  // whose row stride does not depend on the padded rank, up to its own padded rank.
  return for_each_class(P.n, (hipStream_t)stream, [&](int c, hipStream_t cs, bool forked) {
    return lora_bwd_class(&P.d[c], P, c, dy, lddy, x, ldx, h, dx, lddx, grad_A, grad_B, accumulate,
                          (char*)ws + P.ws_off[c], cs, !forked);
  });
}

// ---- packed experts: grouped base GEMM (+ LoRA term) ---------------------------------------------------------------

static bool grouped_desc_ok(const tk_grouped_desc* g) {
  return g && g->rows >= 0 && g->num_groups > 0 && g->groups_per_expert > 0 &&
         g->num_groups % g->groups_per_expert == 0 && g->in_features > 0 && g->out_features > 0;
}

struct GroupedLayout {
  int64_t off_plan, off_count, total;
  GroupedLayout(const tk_grouped_desc& g) {
    SegLayout L(g.rows, g.num_groups);
    int64_t o = 0;
    off_count = o;  o += 256;
    off_plan = o;   o += round_up(grouped_plan_entries(L, g.num_groups / g.groups_per_expert) * (int64_t)sizeof(GroupedPlanEntry), 256);
    total = o;
  }
};

int64_t tk_grouped_linear_workspace_bytes(const tk_grouped_desc* g) {
  if (!grouped_desc_ok(g)) return TK_ERR_INVALID;
  return GroupedLayout(*g).total;
}

int tk_grouped_linear(const tk_grouped_desc* g, const tk_lora_desc* lora, const void* x, int64_t ldx, void* y,
                      int64_t ldy, const void* h, void* ws, int64_t ws_bytes, tk_stream_t stream) {
  if (!grouped_desc_ok(g) || !g->seg_ws || !g->weight_device) return TK_ERR_INVALID;
  if (g->rows == 0) return TK_OK;
  if (g->weight_layout != 0 && g->weight_layout != 1) return TK_ERR_INVALID;
  const int64_t w_rows = g->weight_layout ? g->in_features : g->out_features;
  const int64_t w_cols = g->weight_layout ? g->out_features : g->in_features;
  if (!x || !y || !ws || ldx < g->in_features || ldy < g->out_features || g->ldw < w_cols) return TK_ERR_INVALID;
  if (g->weight_stride < (w_rows - 1) * g->ldw + w_cols) return TK_ERR_INVALID;
  if (g->weight_layout && lora && lora->max_rank > 0) return TK_ERR_INVALID;
  const GroupedLayout W(*g);
  if (ws_bytes < W.total) return TK_ERR_WORKSPACE;
  if (g->dtype != TK_DTYPE_BF16 || force_generic()) return TK_ERR_UNSUPPORTED;
  GroupedArgs a{};
  a.x = (const uint16_t*)x;  a.ldx = ldx;
  a.w = (const uint16_t*)g->weight_device;  a.w_stride = g->weight_stride;  a.ldw = g->ldw;
  a.y = (uint16_t*)y;  a.ldy = ldy;
  a.K = g->in_features;  a.N = g->out_features;  a.src_rows = (int32_t)g->rows;  a.map_rows = g->map_rows;
  a.w_rows_are_inputs = g->weight_layout;
  a.tb = table_bounds(SegLayout(g->rows, g->num_groups));
  if (lora && lora->max_rank > 0) {
    if (!desc_ok(lora) || !h) return TK_ERR_INVALID;
    if (lora->rows != g->rows || lora->num_groups != g->num_groups || lora->in_features != g->in_features ||
        lora->out_features != g->out_features || lora->dtype != g->dtype || lora->seg_ws != g->seg_ws ||
        lora->map_rows != g->map_rows)
      return TK_ERR_INVALID;
    if (lora->max_rank > 64) return TK_ERR_UNSUPPORTED;
    a.rpad = rank_pad(lora->max_rank);
    tk_lora_desc staged;
    if (mixed_weights(*lora)) {
      // fp32 adapters: the epilogue multiplies with the bf16 copy of B, made in the tail of h like tk_lora_expand
      // makes it (tk_lora_shrink left the copy of A there)
      const int rc = stage_weights(lora, (char*)const_cast<void*>(h) + h_core_bytes(lora), false, true,
                                   (hipStream_t)stream, &staged);
      if (rc != TK_OK) return rc;
      lora = &staged;
    }
    a.lora_B = lora->lora_B;  a.ldb = lora->ldb;  a.rank = lora->rank;
    a.hrow = (const uint16_t*)h + (int64_t)a.rpad * h_ld(g->rows, g->num_groups);  // slot-major half of h
  }
  if (!grouped_gemm_supported(a)) return TK_ERR_UNSUPPORTED;
  SegLayout L(g->rows, g->num_groups);
  SegView V(g->seg_ws, L);
  char* w = (char*)ws;
  return launch_grouped_gemm(a, g->num_groups / g->groups_per_expert, g->groups_per_expert,
                             (GroupedPlanEntry*)(w + W.off_plan), (int32_t*)(w + W.off_count), V, L,
                             (hipStream_t)stream);
}

// ---- gated activation ---------------------------------------------------------------------------------------------

int tk_swiglu_fwd(const void* gu, int64_t ld_in, void* out, int64_t ld_out, int64_t rows, int32_t inter, int32_t dtype,
                  tk_stream_t stream) {
  if (rows < 0 || inter <= 0 || (dtype != TK_DTYPE_F32 && dtype != TK_DTYPE_BF16)) return TK_ERR_INVALID;
  if (rows == 0) return TK_OK;
  if (!gu || !out || ld_in < 2 * (int64_t)inter || ld_out < inter) return TK_ERR_INVALID;
  return launch_swiglu(gu, ld_in, nullptr, 0, out, ld_out, rows, inter, dtype, (hipStream_t)stream);
}

int tk_swiglu_bwd(const void* gu, int64_t ld_in, const void* dout, int64_t ld_dout, void* dgu, int64_t ld_dgu,
                  int64_t rows, int32_t inter, int32_t dtype, tk_stream_t stream) {
  if (rows < 0 || inter <= 0 || (dtype != TK_DTYPE_F32 && dtype != TK_DTYPE_BF16)) return TK_ERR_INVALID;
  if (rows == 0) return TK_OK;
  if (!gu || !dout || !dgu || ld_in < 2 * (int64_t)inter || ld_dout < inter || ld_dgu < 2 * (int64_t)inter)
    return TK_ERR_INVALID;
  return launch_swiglu(gu, ld_in, dout, ld_dout, dgu, ld_dgu, rows, inter, dtype, (hipStream_t)stream);
}

// ---- projections that share their input ------------------------------------------------------------------------

// fp32 adapters under bf16 activations are served by the shared kernels when every projection of the call has them
// (or none has): the forward reads the bf16 copies it makes in the tail of every h, the backward reads the fp32
// matrices where the single-projection kernels do and writes fp32 gradients
static bool weights_agree(const tk_lora_desc* const* descs, int32_t n) {
  for (int p = 1; p < n; ++p)
    if ((descs[p]->weights_f32 != 0) != (descs[0]->weights_f32 != 0)) return false;
  return true;
}

static bool shared_descs_ok(const tk_lora_desc* const* descs, int32_t n) {
  if (!descs || n < 1 || n > TK_MAX_SHARED) return false;
  for (int p = 0; p < n; ++p) {
    if (!desc_ok(descs[p])) return false;
    const tk_lora_desc *a = descs[0], *b = descs[p];
    if (a->rows != b->rows || a->in_features != b->in_features || a->num_groups != b->num_groups ||
        a->dtype != b->dtype || a->map_rows != b->map_rows || a->seg_ws != b->seg_ws)
      return false;
  }
  return true;
}

// the kernels of kernels_shared.hip apply: bf16, 2..4 projections of padded rank 16, a split shrink
static bool shared_fast_path(const tk_lora_desc* const* descs, int32_t n) {
  if (n < 2 || descs[0]->dtype != TK_DTYPE_BF16 || force_generic() || !weights_agree(descs, n)) return false;
  for (int p = 0; p < n; ++p)
    if (descs[p]->max_rank < 1 || descs[p]->max_rank > 16) return false;
  return shrink_kslices(descs[0]->in_features, 16) > 1;
}

// ... or the multi-projection launches of the kernels of padded rank 32 / 64: bf16, 2..4 projections whose padded
// ranks agree (and exceed 16)
static bool shared_wide_path(const tk_lora_desc* const* descs, int32_t n) {
  if (n < 2 || descs[0]->dtype != TK_DTYPE_BF16 || force_generic() || !weights_agree(descs, n)) return false;
  const int rpad = rank_pad(descs[0]->max_rank);
  if (rpad != 32 && rpad != 64) return false;
  for (int p = 0; p < n; ++p)
    if (descs[p]->max_rank < 1 || rank_pad(descs[p]->max_rank) != rpad) return false;
  return true;
}

// The shared-input entry points work with one rank class per projection (one layout of h, whatever runs below).
struct SingleClassDescs {
  tk_lora_desc d[TK_MAX_SHARED];
  const tk_lora_desc* p[TK_MAX_SHARED];
  SingleClassDescs(const tk_lora_desc* const* descs, int32_t n) {
    for (int i = 0; i < TK_MAX_SHARED; ++i) {
      p[i] = nullptr;
      if (descs && i < n && descs[i]) {
        d[i] = *descs[i];
        d[i].rank_classes = 0;
        p[i] = &d[i];
      }
    }
  }
};

int tk_lora_fwd_shared(const tk_lora_desc* const* descs_in, int32_t n, const void* x, int64_t ldx, void* const* y,
                       const int64_t* ldy, void* const* h, tk_stream_t stream) {
  const SingleClassDescs local(descs_in, n);
  const tk_lora_desc* const* descs = descs_in ? local.p : nullptr;
  if (!shared_descs_ok(descs, n) || !y || !ldy || !h) return TK_ERR_INVALID;
  const tk_lora_desc* d0 = descs[0];
  if (d0->rows == 0) return TK_OK;
  if (!x || ldx < d0->in_features) return TK_ERR_INVALID;
  for (int p = 0; p < n; ++p)
    if (!y[p] || !h[p] || ldy[p] < descs[p]->out_features) return TK_ERR_INVALID;
  hipStream_t s = (hipStream_t)stream;
  SegLayout L(d0->rows, d0->num_groups);
  SegView V(d0->seg_ws, L);
  PassArgs a[TK_MAX_SHARED] = {};
  bool fast = shared_fast_path(descs, n);
  bool wide = !fast && shared_wide_path(descs, n);
  int rc;
  // fp32 adapters: the shared kernels read bf16 copies, made here in the tail of every projection's h (where
  // tk_lora_fwd makes them); `kd` are the descriptors the kernels work from
  tk_lora_desc staged[TK_MAX_SHARED];
  const tk_lora_desc* kd[TK_MAX_SHARED];
  for (int p = 0; p < n; ++p) kd[p] = descs[p];
  if ((fast || wide) && mixed_weights(*d0)) {  // (all projections alike: weights_agree) one launch converts them all
    void* stage[TK_MAX_SHARED];
    for (int p = 0; p < n; ++p) stage[p] = (char*)h[p] + h_core_bytes(descs[p]);
    if ((rc = launch_convert_weights_multi(descs, stage, n, true, true, s)) != TK_OK) return rc;
    for (int p = 0; p < n; ++p) {
      staged_desc(descs[p], stage[p], &staged[p]);
      kd[p] = &staged[p];
    }
  }
  for (int p = 0; p < n; ++p) {
    a[p] = fwd_pass_args(kd[p], x, ldx, y[p], ldy[p], h[p]);
    fast = fast && pass_mfma_supported(a[p]);
  }
  if (!fast) {
    for (int p = 0; p < n && wide; ++p) wide = pass_mfma_supported(a[p]) && a[p].kslices == a[0].kslices;
    if (wide) {
      // every projection's shrink in one launch, the pieces of x crossing memory once; then y_p += h_p B_p^T
      if ((rc = launch_shrink_multi(a, n, V, L, s)) != TK_OK) return rc;
      for (int p = 0; p < n; ++p)
        if ((rc = launch_pass_mfma(a[p], V, L, 2, s)) != TK_OK) return rc;
      return TK_OK;
    }
    for (int p = 0; p < n; ++p)
      if ((rc = tk_lora_fwd(descs[p], x, ldx, y[p], ldy[p], h[p], stream)) != TK_OK) return rc;
    return TK_OK;
  }
  SharedShrinkArgs sa{};
  sa.src = x;  sa.ld_src = ldx;
  sa.width_src = d0->in_features;  sa.src_rows = (int32_t)d0->rows;  sa.map_rows = d0->map_rows;
  sa.kslices = a[0].kslices;  sa.nproj = n;
  sa.tb = a[0].tb;
  for (int p = 0; p < n; ++p) {
    sa.w[p] = kd[p]->lora_A;  sa.ld_w[p] = kd[p]->lda;
    sa.rank[p] = kd[p]->rank;  sa.hpart[p] = a[p].hpart;
  }
  if ((rc = launch_shrink_shared(sa, V, L, s)) != TK_OK) return rc;
  // every projection in one launch each: add the slices (h_p), then y_p += h_p B_p^T
  return launch_pass_multi(a, n, V, L, 4 | 2, s);
}

int tk_lora_bwd_shared(const tk_lora_desc* const* descs_in, int32_t n, const void* const* dy, const int64_t* lddy,
                       const void* x, int64_t ldx, const void* const* h, void* dx, int64_t lddx,
                       void* const* const* grad_A, void* const* const* grad_B, int32_t accumulate, void* const* ws,
                       const int64_t* ws_bytes, tk_stream_t stream) {
  const SingleClassDescs local(descs_in, n);
  const tk_lora_desc* const* descs = descs_in ? local.p : nullptr;
  if (!shared_descs_ok(descs, n) || !dy || !lddy || !h || !grad_A || !grad_B || !ws || !ws_bytes) return TK_ERR_INVALID;
  const tk_lora_desc* d0 = descs[0];
  if (d0->rows == 0) return TK_OK;
  if (!x || ldx < d0->in_features || !dx || lddx < d0->in_features) return TK_ERR_INVALID;
  hipStream_t s = (hipStream_t)stream;
  SegLayout L(d0->rows, d0->num_groups);
  SegView V(d0->seg_ws, L);
  BwdPlan plan[TK_MAX_SHARED];
  bool fast = shared_fast_path(descs, n);
  for (int p = 0; p < n; ++p) {
    const tk_lora_desc* d = descs[p];
    if (!dy[p] || lddy[p] < d->out_features || !h[p] || !grad_A[p] || !grad_B[p] || !ws[p]) return TK_ERR_INVALID;
    BwdLayout B(*d);
    if (ws_bytes[p] < B.total) return TK_ERR_WORKSPACE;
    if (d->max_rank == 0) {
      fast = false;
      continue;
    }
    plan[p] = bwd_plan(d, B, dy[p], lddy[p], x, ldx, h[p], dx, lddx, grad_A[p], grad_B[p], accumulate, ws[p]);
    fast = fast && pass_mfma_supported(plan[p].a) && dy_fused_supported(plan[p].gb, plan[p].a.kslices) &&
           wgrad_mfma_supported(plan[p].ga);
  }
  int rc;
  if (!fast) {
    bool wide = shared_wide_path(descs, n);
    for (int p = 0; p < n && wide; ++p)
      wide = pass_mfma_supported(plan[p].a) && wgrad_mfma_supported(plan[p].ga) && wgrad_mfma_supported(plan[p].gb) &&
             descs[p]->out_features % 8 == 0;
    if (wide) {
      // Per projection what only it touches (its dy: the transposed weight copies, dh_p = s dy_p B_p and dB_p), then
      // once for all of them what touches the shared tensors: dx += sum_p dh_p A_p in one read-modify-write, and
      // every dA_p = dh_p^T x from launches that fetch each tile of x once.
      const int rpad = plan[0].a.rpad;
      SharedExpandArgs ea{};
      ea.dst = dx;  ea.ld_dst = lddx;  ea.width_dst = d0->in_features;  ea.map_rows = d0->map_rows;  ea.nproj = n;
      ea.tb = table_bounds(L);
      SharedWgradArgs wa{};
      wa.nproj = n;
      WgradArgs red[2 * TK_MAX_SHARED] = {};
      for (int p = 0; p < n; ++p) {
        BwdPlan& P = plan[p];
        const int fused_ks = fused_dy_kslices(descs[p]->out_features, rpad);
        if (fused_ks && dy_fused_supported(P.gb, fused_ks)) {  // one pass over dy_p: dB_p, the slices of dh_p, A_p^T
          P.a.kslices = fused_ks;
          WgradArgs gb = P.gb;
          gb.tr = P.tr;
          gb.tr.bT = nullptr;
          if ((rc = launch_dy_fused(gb, descs[p]->lora_B, descs[p]->ldb, P.a.hpart, fused_ks, V, L, s)) != TK_OK)
            return rc;
          if ((rc = launch_pass_mfma(P.a, V, L, 4, s)) != TK_OK) return rc;
        } else {
          if ((rc = launch_transpose_job(P.tr, descs[p]->rank, rpad, s)) != TK_OK) return rc;
          if ((rc = launch_pass_mfma(P.a, V, L, 1, s)) != TK_OK) return rc;
          if ((rc = launch_wgrad_mfma(P.gb, V, L, s)) != TK_OK) return rc;
        }
        ea.hrow[p] = (const char*)P.dh + (int64_t)rpad * P.a.ldh * 2;  // slot-major half of the dh buffer (bf16)
        ea.aT[p] = P.aT;
        ea.rank[p] = descs[p]->rank;
        wa.w[p] = P.ga;
        red[2 * p] = P.ga;
        red[2 * p + 1] = P.gb;
      }
      if ((rc = launch_expand_shared_wide(ea, rpad, V, L, s)) != TK_OK) return rc;
      if ((rc = launch_wgrad_coop_multi(wa, V, L, s)) != TK_OK) return rc;
      return launch_wgrad_reduce_multi(red, 2 * n, V, L, s);
    }
    for (int p = 0; p < n; ++p)
      if ((rc = tk_lora_bwd(descs[p], dy[p], lddy[p], x, ldx, h[p], dx, lddx, grad_A[p], grad_B[p], accumulate, ws[p],
                            ws_bytes[p], stream)) != TK_OK)
        return rc;
    return TK_OK;
  }
  SharedExpandArgs ea{};
  ea.dst = dx;  ea.ld_dst = lddx;  ea.width_dst = d0->in_features;  ea.map_rows = d0->map_rows;  ea.nproj = n;
  ea.tb = table_bounds(L);
  SharedWgradArgs wa{};
  wa.nproj = n;
  DyFusedJob dj[TK_MAX_SHARED] = {};
  PassArgs pa[TK_MAX_SHARED] = {};
  WgradArgs red[2 * TK_MAX_SHARED] = {};
  for (int p = 0; p < n; ++p) {
    BwdPlan& P = plan[p];
    dj[p].a = P.gb;
    dj[p].a.tr = P.tr;
    dj[p].a.tr.bT = nullptr;  // the fused kernel reads B_p where it lies
    dj[p].a.tr.swizzle_a = 1;
    dj[p].lora_B = descs[p]->lora_B;  dj[p].ldb = descs[p]->ldb;
    dj[p].hpart = P.a.hpart;  dj[p].kslices = P.a.kslices;
    pa[p] = P.a;
    ea.hrow[p] = (const char*)P.dh + (int64_t)P.a.rpad * P.a.ldh * 2;  // slot-major half of the dh buffer (bf16)
    ea.aT[p] = P.aT;
    ea.rank[p] = descs[p]->rank;
    wa.w[p] = P.ga;
    red[2 * p] = P.ga;
    red[2 * p + 1] = P.gb;
  }
  // every dy_p once: dB_p, the slices of dh_p and the A_p^T copies; then every dh_p
  if ((rc = launch_dy_fused_multi(dj, n, V, L, s)) != TK_OK) return rc;
  if ((rc = launch_pass_multi(pa, n, V, L, 4, s)) != TK_OK) return rc;
  if ((rc = launch_expand_shared(ea, V, L, s)) != TK_OK) return rc;  // dx += sum_p dh_p A_p
  if ((rc = launch_wgrad_shared(wa, V, L, s)) != TK_OK) return rc;   // dA_p for all p, x read once
  return launch_wgrad_reduce_multi(red, 2 * n, V, L, s);
}

int64_t tk_opt_workspace_bytes(int32_t num_tensors, int64_t max_numel) {
  if (num_tensors < 0 || max_numel < 0) return TK_ERR_INVALID;
  return round_up(4 * opt_partial_floats(num_tensors, max_numel) + 4, 256);
}

static bool opt_args_ok(const tk_opt_tensor* tensors, int32_t num_tensors, const tk_opt_tenant* tenants,
                        int32_t num_tenants, int64_t max_numel, int32_t dtype) {
  if (num_tensors < 0 || num_tenants <= 0 || max_numel < 0) return false;
  if (num_tensors > 0 && (!tensors || !tenants)) return false;
  if (num_tensors > 65535) return false;  // grid.y
  return dtype == TK_DTYPE_F32 || dtype == TK_DTYPE_BF16;
}

int tk_opt_grad_norm(const tk_opt_tensor* tensors, int32_t num_tensors, const tk_opt_tenant* tenants,
                     int32_t num_tenants, int64_t max_numel, int32_t dtype, float* norm_out, float* clip_out,
                     void* ws, int64_t ws_bytes, tk_stream_t stream) {
  if (!opt_args_ok(tensors, num_tensors, tenants, num_tenants, max_numel, dtype) || !tenants || !norm_out || !clip_out)
    return TK_ERR_INVALID;
  if (!ws || ws_bytes < tk_opt_workspace_bytes(num_tensors, max_numel)) return TK_ERR_WORKSPACE;
  return launch_opt_grad_norm(tensors, num_tensors, tenants, num_tenants, max_numel > 0 ? max_numel : 1, dtype, norm_out,
                              clip_out, (float*)ws, (hipStream_t)stream);
}

int tk_opt_adamw_step(const tk_opt_tensor* tensors, int32_t num_tensors, const tk_opt_tenant* tenants,
                      int32_t num_tenants, int64_t max_numel, int32_t dtype, const float* clip, int32_t flags,
                      tk_stream_t stream) {
  if (!opt_args_ok(tensors, num_tensors, tenants, num_tenants, max_numel, dtype)) return TK_ERR_INVALID;
  if (num_tensors == 0 || max_numel == 0) return TK_OK;
  return launch_opt_adamw(tensors, num_tensors, tenants, max_numel, dtype, clip, flags, (hipStream_t)stream);
}

}  // extern "C"
