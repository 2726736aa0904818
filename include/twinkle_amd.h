/*
 * twinkle_amd — C ABI of the MI355X (gfx950) multi-LoRA hot path.
 *
 * Plain pointers and sizes only; every pointer named "device" is HIP device
 * memory owned by the caller.  All work is ordered on the stream that is
 * passed in (a hipStream_t cast to void*; NULL = the null stream).  No call
 * allocates, frees, synchronises the device or keeps state between calls,
 * except where stated (tk_lora_fwd_noalloc keeps a scratch buffer per GPU).  Return value: TK_OK or a negative TK_ERR_* code.
 *
 * Host threads: every entry point may be called from any thread.  The one
 * per-device resource the library keeps (the side stream of tk_lora_bwd and
 * its events) is guarded, so concurrent calls on one device are enqueued one
 * after the other; what they compute may still overlap on the GPU only as
 * far as their streams allow, and two calls that share a workspace, an h
 * buffer or gradient tensors must be ordered by the caller.
 *
 * The reference (modelscope/twinkle) is pure Python and has no FFI for this
 * path; each entry point below names the reference code whose work it takes
 * over (paths relative to the reference checkout).
 */
#ifndef TWINKLE_AMD_H
#define TWINKLE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* tk_stream_t; /* hipStream_t */

enum {
  TK_OK = 0,
  TK_ERR_INVALID = -1,     /* bad argument (null pointer, negative size, misaligned stride) */
  TK_ERR_WORKSPACE = -2,   /* workspace smaller than the matching *_bytes() query */
  TK_ERR_UNSUPPORTED = -3, /* shape outside what the kernels handle (see each call) */
  TK_ERR_LAUNCH = -4,      /* HIP reported an error at launch */
  TK_ERR_SCRATCH = -5      /* tk_lora_fwd_noalloc: the problem needs more than TK_NOALLOC_SCRATCH_BYTES */
};

enum { TK_DTYPE_F32 = 0, TK_DTYPE_BF16 = 1 };
enum { TK_KEY_I32 = 0, TK_KEY_I64 = 1 };

/* Rows per forward tile and per smallest weight-gradient chunk (fixed at build time; chunks grow with the
 * batch, about 32 of them over all rows: 128 rows up to 4096 rows, 512 at 16384, up to 4096). */
#define TK_TILE_ROWS 32
#ifndef TK_CHUNK_ROWS
#define TK_CHUNK_ROWS 128
#endif
#define TK_MAX_GROUPS 16384
#define TK_MAX_RANK 128

const char* tk_version(void);
const char* tk_error_string(int code);

/* ---------------------------------------------------------------------------
 * Segment builder: rows -> groups, stable.
 *
 * Replaces the reference's mask-based ordering
 *   src/twinkle/model/transformers/moe/expert_parallel.py:254-255 (one_hot mask),
 *   src/twinkle/model/transformers/moe/ep_utils.py:99-118 (masked_select order),
 *   src/twinkle/model/transformers/moe/ep_utils.py:191 (per-group counts),
 *   src/twinkle/model/transformers/moe/expert_parallel.py:347-349 (host cumsum
 *   with .item() syncs),
 * and widens MultiLora.adapter()'s one-adapter-per-call selection
 *   (src/twinkle/model/multi_lora.py:126-163) to one adapter id per row.
 *
 * keys[f] in [0, num_groups) is the group of flat row f (top-k routing: f = k*T + t).
 * perm_out[j]  = flat row placed at sorted position j (stable: ties keep ascending f),
 * offsets_out[g] = first sorted position of group g, offsets_out[num_groups] = rows that have a group.
 * Both are int64 like the reference's tensors and may be NULL when only the
 * workspace is wanted.  seg_ws receives the device-side segment table the
 * LoRA and permute calls read; it must stay alive and unmodified while they run.
 * A key outside [0, num_groups) (say -1 for a padding row) gives its row no group: the row is
 * placed after the last group in perm_out (stable among such rows) and no LoRA or grouped-GEMM call
 * reads or writes it; tk_permute_rows / tk_unpermute_rows move it like any other row.
 * tk_segment_bad_keys() reports how many such keys there were.
 * Limits: num_groups <= TK_MAX_GROUPS, rows < 2^31.
 * ------------------------------------------------------------------------ */
int64_t tk_segment_workspace_bytes(int64_t rows, int32_t num_groups);
int tk_segment_build(const void* keys_device, int32_t key_dtype, int64_t rows, int32_t num_groups,
                     int64_t* perm_out_device, int64_t* offsets_out_device, void* seg_ws_device,
                     int64_t seg_ws_bytes, tk_stream_t stream);
/* Synchronises the stream and copies one counter back: number of out-of-range keys. */
int tk_segment_bad_keys(const void* seg_ws_device, tk_stream_t stream, int64_t* count_out_host);

/* Checks a segment table on the host (a debugging and test aid; no counterpart in the reference): copies the whole
 * workspace back (synchronises the stream) and rebuilds every array from the group sizes and the row order it holds.
 * TK_OK when every entry is what tk_segment_build writes for some keys of (rows, num_groups): every row in exactly one
 * slot, rows ascending inside a group, group / tile / chunk / partial numbers inside the table's bounds and consistent
 * with each other.  Otherwise TK_ERR_INVALID, with the number of the first failing check (1 header, 2 offsets, 3 first
 * tiles, 4 group of a tile, 5 slot rows / positions, 6 permutation and its inverse, 7 stable order, 8 walk orders,
 * 9 chunks, 10 first chunks / partial slots) and the index it failed at in the two outputs (either may be NULL).
 * The kernels themselves compare every table entry they index with against the table's bounds and skip what lies
 * outside, so a table that was overwritten gives wrong results, not accesses outside the caller's tensors; this
 * call is how to find out that it was. */
int tk_segment_validate(const void* seg_ws_device, int64_t rows, int32_t num_groups, tk_stream_t stream,
                        int32_t* failed_check_out_host, int64_t* index_out_host);

/* ---------------------------------------------------------------------------
 * Row gather / weighted scatter-back in segment order.
 *
 * tk_permute_rows replaces ep_utils.py:99-118 (`permute`: index_select by the
 * masked_select order): dst[j] = src[perm[j] mod num_tokens] (* w[token, k] when
 * weights is non-NULL; that form is the backward of tk_unpermute_rows).
 * tk_unpermute_rows replaces ep_utils.py:121-149 / :280-287 (`unpermute`:
 * zero-init + scatter_add_ with routing weights):
 *   out[t] = sum_{k ascending} rows[pos(k*T + t)] * w[t, k]
 * computed as a gather with a fixed summation order (deterministic, unlike
 * the reference's atomics).  weights is [num_tokens, top_k] in `dtype`, or NULL
 * for unit weights.  rows == num_tokens * top_k.
 * ------------------------------------------------------------------------ */
int tk_permute_rows(const void* src_device, int64_t ld_src, void* dst_device, int64_t ld_dst,
                    const void* weights_device, const void* seg_ws_device, int64_t rows, int64_t num_tokens,
                    int32_t width, int32_t num_groups, int32_t dtype, tk_stream_t stream);
int tk_unpermute_rows(const void* rows_device, int64_t ld_rows, void* out_device, int64_t ld_out,
                      const void* weights_device, const void* seg_ws_device, int64_t rows, int64_t num_tokens,
                      int32_t width, int32_t num_groups, int32_t dtype, tk_stream_t stream);
/* dw[t, k] = <dout[t, :], rows[pos(k*T + t), :]>   (gradient of the routing weights, fp32 out) */
int tk_unpermute_weight_grad(const void* dout_device, int64_t ld_dout, const void* rows_device, int64_t ld_rows,
                             float* dw_device, const void* seg_ws_device, int64_t rows, int64_t num_tokens,
                             int32_t width, int32_t num_groups, int32_t dtype, tk_stream_t stream);

/* ---------------------------------------------------------------------------
 * Segmented LoRA linear.
 *
 * Replaces the body of the patched LoraLayer forward
 *   src/twinkle/model/multi_lora.py:315-326
 *     h = linear(x, A[:r]); u = linear(h, B[:, :r]); result = result + u * scaling
 * and the autograd of those two F.linear calls, for every adapter of a mixed
 * batch in one pass; and, with per-(expert, tenant) groups, the effect of the
 * merged expert weights of
 *   src/twinkle/model/multi_lora_target_parameters.py:158-179 inside the per-expert loop
 *   src/twinkle/model/transformers/moe/expert_parallel.py:347-371
 * without materialising the [E, out, in] delta.
 *
 * Group g uses A_g = lora_A[g] ([>= rank[g], in_features], row stride lda) and
 * B_g = lora_B[g] ([out_features, >= rank[g]], row stride ldb): the slot
 * tensors of the reference at their physical strides; only the leading
 * rank[g] rows / columns are read or written.  rank[g] == 0 skips the group.
 * ------------------------------------------------------------------------ */
typedef struct tk_lora_desc {
  int64_t rows;         /* rows covered by the segment table */
  int32_t in_features;  /* K */
  int32_t out_features; /* M */
  int32_t num_groups;   /* G, as given to tk_segment_build */
  int32_t max_rank;     /* host-side upper bound of rank[g], <= TK_MAX_RANK */
  int32_t dtype;        /* TK_DTYPE_* of x, y, A, B, h and the gradients */
  int32_t map_rows;     /* 1: sorted position p touches row perm[p] of x / y (dense LoRA);
                           0: rows are already in segment order (after tk_permute_rows) */
  const void* seg_ws;          /* device, from tk_segment_build */
  const void* const* lora_A;   /* device array [G] of device pointers */
  const void* const* lora_B;   /* device array [G] of device pointers */
  int64_t lda;                 /* elements */
  int64_t ldb;                 /* elements */
  const int32_t* rank;         /* device [G] */
  const float* scale;          /* device [G]: alpha/r or alpha/sqrt(r) */
  int32_t weights_f32;         /* 1 with dtype TK_DTYPE_BF16: A, B and their gradients are fp32 (lda, ldb in fp32
                                  elements) while x, y and h are bf16, the usual state of a PEFT model whose base is
                                  bf16 (adapters are kept in fp32; src/twinkle/model/multi_lora.py:320 casts x to
                                  their dtype).  The kernels read bf16 copies of A and B that every call makes on
                                  the fly inside h / the backward workspace (round to nearest even), multiply on
                                  the matrix cores with fp32 accumulation and write fp32 gradients.  0: A, B and
                                  the gradients have `dtype`.  The shared-input entry points take it when all their
                                  projections agree (else they run one call per projection), tk_grouped_linear
                                  converts B into the tail of h like tk_lora_expand.  The backward reads only the
                                  part of h in front of those copies. */
  int32_t rank_classes;        /* Which padded ranks occur among rank[] (which lives on the device, so the host
                                  says it here): bit 0 = some group has rank 1..16, bit 1 = 17..32, bit 2 = 33..64,
                                  bit 3 = 65..128; the bit of max_rank's class must be among them.  With more than
                                  one bit set, tk_lora_bwd runs each class of groups on the kernels of its own
                                  padded rank (a tenant of rank 8 next to one of rank 64 is not padded to 64: every
                                  tenant carries its own r, src/twinkle/model/multi_lora.py:318-325), the classes
                                  side by side on streams of the library, and the backward workspace holds one
                                  region per class (tk_lora_bwd_workspace_bytes accounts for it).  A group whose
                                  rank lies in a class that is not listed is served by the next listed class above
                                  it, so a mask may be too coarse but loses no group.  The
                                  forward and the layout of h do not depend on the field.  0 (or one bit): one
                                  class for all groups, padded to max_rank.  The shared-input entry points ignore
                                  the field. */
} tk_lora_desc;

/* Bytes of the saved shrink output h (scale * x A^T per row, kept for backward). */
int64_t tk_lora_h_bytes(const tk_lora_desc* desc);
int64_t tk_lora_bwd_workspace_bytes(const tk_lora_desc* desc);

/* y[row] += scale_g * (x[row] A_g^T) B_g^T in place on the base output; h_device is written. */
int tk_lora_fwd(const tk_lora_desc* desc, const void* x_device, int64_t ldx, void* y_device, int64_t ldy,
                void* h_device, tk_stream_t stream);

/* tk_lora_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same result as tk_lora_fwd, bit for bit: y is
 * updated in place; the shrink output, which tk_lora_fwd leaves in the caller's h buffer for the backward pass, goes
 * to a buffer of TK_NOALLOC_SCRATCH_BYTES that the library holds in every GPU's memory from the first call on that
 * GPU until the process ends, so there is no backward after this call (inference and evaluation passes).  The call
 * allocates and frees nothing and does not synchronise.  TK_ERR_SCRATCH when tk_lora_h_bytes(desc) exceeds
 * TK_NOALLOC_SCRATCH_BYTES (16 MiB: up to 16384 rows at in_features 4096 for any rank up to 64).  All calls on one
 * GPU share that GPU's buffer and it keeps the last call's contents: two calls whose execution may overlap on one
 * GPU (different streams, or different host threads without ordering) race; order them on one stream.
 * The first call on a GPU looks up the buffer's device address (hipGetSymbolAddress, which may load the library's
 * device code for that GPU): make one call per GPU outside any stream capture before capturing this entry point;
 * every later call on that GPU only enqueues kernels. */
#define TK_NOALLOC_SCRATCH_BYTES (16 << 20)
int tk_lora_fwd_noalloc(const tk_lora_desc* desc, const void* x_device, int64_t ldx, void* y_device, int64_t ldy,
                        tk_stream_t stream);

/* The two halves of tk_lora_fwd, for callers that time or schedule them separately:
 * tk_lora_shrink writes h = scale_g * x A_g^T (reference: multi_lora.py:322-323, the first F.linear),
 * tk_lora_expand adds h B_g^T onto y in place (reference: multi_lora.py:324-326). */
int tk_lora_shrink(const tk_lora_desc* desc, const void* x_device, int64_t ldx, void* h_device, tk_stream_t stream);
int tk_lora_expand(const tk_lora_desc* desc, const void* h_device, void* y_device, int64_t ldy, tk_stream_t stream);

/* dx[row] += scale_g * (dy[row] B_g) A_g        (skipped when dx_device is NULL)
 * dA_g[:r] (+)= (scale_g * dy B_g)^T x          (skipped when grad_A is NULL)
 * dB_g[:, :r] (+)= dy^T h                       (skipped when grad_B is NULL)
 * grad_A / grad_B are device arrays [G] of device pointers with the strides lda / ldb;
 * accumulate != 0 adds onto their contents, 0 overwrites the live [:r] block.  Elements
 * outside the live block are never touched.  Weight gradients are reduced over
 * row chunks in a fixed order: results are bitwise repeatable. */
int tk_lora_bwd(const tk_lora_desc* desc, const void* dy_device, int64_t lddy, const void* x_device, int64_t ldx,
                const void* h_device, void* dx_device, int64_t lddx, void* const* grad_A, void* const* grad_B,
                int32_t accumulate, void* workspace_device, int64_t workspace_bytes, tk_stream_t stream);

/* ---------------------------------------------------------------------------
 * Multi-tenant optimizer step over adapter tensors (one launch set for all tenants).
 *
 * What the reference does per tenant, one tenant at a time (src/twinkle/model/transformers/transformers.py):
 * clip_grad_norm (:732-778) divides the tenant's gradients by its token count and clips their total norm
 * (src/twinkle/utils/grad_clip.py:31-96, torch.nn.utils.clip_grad_norm_ on one GPU), step (:835-876) runs
 * torch.optim.AdamW / Adam with per-call lr / weight_decay / eps / betas, zero_grad (:879-894) clears the
 * gradients.  Here every tensor carries its tenant's index and the tenants' numbers sit in one table.
 * ------------------------------------------------------------------------- */
typedef struct tk_opt_tensor { /* one contiguous parameter tensor of one tenant (device pointers) */
  void* param;                 /* dtype given per call */
  void* grad;                  /* same dtype and size */
  float* exp_avg;              /* fp32 first moment, numel floats */
  float* exp_avg_sq;           /* fp32 second moment */
  int64_t numel;
  int32_t tenant;              /* row of the tenant table */
  int32_t reserved;
} tk_opt_tensor;

typedef struct tk_opt_tenant { /* one row of the tenant table */
  float lr, beta1, beta2, eps, weight_decay;
  float one_minus_beta1;       /* 1 - beta1 and 1 - beta2, rounded from double by the caller: formed in fp32 from */
  float one_minus_beta2;       /* the rounded betas they would be off by 1e-5 relative (beta2 = 0.999) */
  float bias_correction1;      /* 1 - beta1^step, computed in double by the caller (as torch does) */
  float bias_correction2_sqrt; /* sqrt(1 - beta2^step) */
  float grad_scale;            /* 1 / num_tokens (grad_clip.py:81-96: gradients are divided by the token count) */
  float max_grad_norm;         /* <= 0: no clipping */
  float norm_type;             /* 2, or +infinity for the max norm */
  int32_t active;              /* 0: the tenant's tensors are skipped (no step for it this time) */
  int32_t reserved;
} tk_opt_tenant;

#define TK_OPT_WRITE_GRADS 1 /* leave the normalised, clipped gradients in grad (what the reference's grads hold) */
#define TK_OPT_ZERO_GRADS 2  /* clear grad in the same pass (the reference's zero_grad after step) */

/* Bytes of scratch for tk_opt_grad_norm. */
int64_t tk_opt_workspace_bytes(int32_t num_tensors, int64_t max_numel);

/* norm_out[t] = norm of tenant t's gradients after division by its token count, before clipping (the value
 * clip_grad_norm returns); clip_out[t] = min(1, max_grad_norm / (norm + 1e-6)), 1 without clipping.  Both are
 * device arrays [num_tenants]; tensors_device / tenants_device are device arrays; no host synchronisation.
 * Sums run in a fixed order: bitwise repeatable. */
int tk_opt_grad_norm(const tk_opt_tensor* tensors_device, int32_t num_tensors, const tk_opt_tenant* tenants_device,
                     int32_t num_tenants, int64_t max_numel, int32_t dtype, float* norm_out, float* clip_out,
                     void* workspace_device, int64_t workspace_bytes, tk_stream_t stream);

/* AdamW (decoupled weight decay; weight_decay = 0 gives Adam) on every active tenant's tensors with
 * g' = grad * grad_scale * clip[t] (clip_device may be NULL: no clipping).  fp32 arithmetic and moments. */
int tk_opt_adamw_step(const tk_opt_tensor* tensors_device, int32_t num_tensors, const tk_opt_tenant* tenants_device,
                      int32_t num_tenants, int64_t max_numel, int32_t dtype, const float* clip_device, int32_t flags,
                      tk_stream_t stream);

/* ---------------------------------------------------------------------------
 * Projections that share their input (q / k / v, gate / up): one call for all of them, with the shared
 * tensors crossing memory once.  Same results contract as one tk_lora_fwd / tk_lora_bwd per projection, which
 * is also what runs when the shapes are outside the shared kernels (bf16, 2..4 projections whose max_rank
 * round up to the same padded rank 16, 32 or 64, in_features a multiple of 1024 .. see the single-projection
 * fast-path limits): forward reads x once instead of once per projection; backward reads x once for all dA
 * and updates dx once with the sum over the projections (one rounding instead of one per projection).  At
 * padded rank 16 the reads of x are shared inside one kernel; at 32 and 64 the projections' blocks that need
 * the same piece of x are launched side by side on one XCD, so the piece comes from memory once and from that
 * L2 afterwards.  The descriptors must agree in rows,
 * in_features, num_groups, dtype, map_rows and seg_ws.  Arrays indexed by projection are host arrays.
 * No counterpart in the reference, which runs every projection's two F.linear calls on its own
 * (multi_lora.py:322-326).
 * ------------------------------------------------------------------------- */
#define TK_MAX_SHARED 4
int tk_lora_fwd_shared(const tk_lora_desc* const* descs, int32_t num_proj, const void* x_device, int64_t ldx,
                       void* const* y_device, const int64_t* ldy, void* const* h_device, tk_stream_t stream);
int tk_lora_bwd_shared(const tk_lora_desc* const* descs, int32_t num_proj, const void* const* dy_device,
                       const int64_t* lddy, const void* x_device, int64_t ldx, const void* const* h_device,
                       void* dx_device, int64_t lddx, void* const* const* grad_A, void* const* const* grad_B,
                       int32_t accumulate, void* const* workspace_device, const int64_t* workspace_bytes,
                       tk_stream_t stream);

/* ---- packed experts: grouped base GEMM with the LoRA term in its epilogue -------------------------------
 *
 * y[row] = x[row] W_e^T (+ h[row] B_g^T) for every row of the segment table, where the table was built from
 * keys g = e * groups_per_expert + tenant and expert e's weight [out_features][in_features] starts at
 * weight_device + e * weight_stride elements (row stride ldw).  Replaces the reference's host loop over the
 * experts (one F.linear per projection and one host synchronisation per expert for the chunk boundaries,
 * moe/expert_parallel.py:347-371) by one launch; with `lora` it also takes over the expert LoRA delta that the
 * reference merges into the weights (multi_lora_target_parameters.py:158-179): call tk_lora_shrink(lora, x, h)
 * first and pass that h here, y is then written once with both terms.  The backward of the base term is the
 * same call with weight_layout = 1 on the same weights (dx = dy W_e, in_features and out_features swapped);
 * the LoRA gradients come from tk_lora_bwd with dx accumulated onto this call's result.
 *
 * bf16 only; in_features a multiple of 64, out_features of 128, ldx / ldw / weight_stride multiples of 8 and
 * ldy of 4 elements, 16-byte aligned x and weight, 8-byte aligned y: anything else is TK_ERR_UNSUPPORTED
 * (run the experts one by one then).  y rows of the table are overwritten; x and y must not overlap.
 * lora (optional) must describe the same rows, groups, features, seg_ws and map_rows. */
typedef struct {
  int64_t rows;
  int32_t num_groups;        /* experts * groups_per_expert */
  int32_t groups_per_expert; /* tenants per expert in the key; 1 for the reference's expert-only grouping */
  int32_t in_features;
  int32_t out_features;
  int32_t dtype;             /* TK_DTYPE_BF16 */
  int32_t map_rows;          /* as in tk_lora_desc */
  const void* seg_ws;        /* device: segment table of tk_segment_build for (rows, num_groups) */
  const void* weight_device;
  int64_t weight_stride;     /* elements between consecutive experts */
  int64_t ldw;
  int32_t weight_layout;     /* 0: [out_features][in_features] per expert (y = x W^T);
                                1: [in_features][out_features] per expert (y = x W): the backward of a layout-0
                                   call on the same memory, dx = dy W.  No LoRA term with layout 1. */
  int32_t reserved;          /* 0 */
} tk_grouped_desc;

int64_t tk_grouped_linear_workspace_bytes(const tk_grouped_desc* desc);
int tk_grouped_linear(const tk_grouped_desc* desc, const tk_lora_desc* lora, const void* x_device, int64_t ldx,
                      void* y_device, int64_t ldy, const void* h_device, void* workspace_device,
                      int64_t workspace_bytes, tk_stream_t stream);

/* ---- gated activation of the packed experts --------------------------------------------------------------
 *
 * hidden[row][c] = silu(gate_up[row][c]) * gate_up[row][inter + c], c < inter: what the reference computes
 * between the two expert projections as `gate, up = gate_up_out.chunk(2, -1); act_fn(gate) * up` with
 * act_fn = SiLU (moe/expert_parallel.py:363-366), in one pass, fp32 arithmetic, one rounding.
 * tk_swiglu_bwd writes d(gate | up) from gate_up and d(hidden).  bf16 or fp32; inter and the row strides
 * multiples of 8 elements, pointers aligned to 8 elements: TK_ERR_UNSUPPORTED otherwise. */
int tk_swiglu_fwd(const void* gate_up_device, int64_t ld_gate_up, void* hidden_device, int64_t ld_hidden,
                  int64_t rows, int32_t inter, int32_t dtype, tk_stream_t stream);
int tk_swiglu_bwd(const void* gate_up_device, int64_t ld_gate_up, const void* dhidden_device, int64_t ld_dhidden,
                  void* dgate_up_device, int64_t ld_dgate_up, int64_t rows, int32_t inter, int32_t dtype,
                  tk_stream_t stream);

/* ---- memory yardsticks ---------------------------------------------------------------------------------------
 *
 * One launch of a kernel that only moves memory in the access pattern of one of the kernels above, over a
 * [rows][width] bf16 buffer `a` (`b`: the destination of TK_YS_COPY, a sink of at least 4 KB otherwise):
 * what bench.py --yardstick times to say how fast this GPU runs each pattern with no arithmetic at all.
 * `row_of` (device, [rows] int32, optional) is a permutation of the rows, taken 32 entries per tile like the
 * segment table's slots; NULL takes the rows in order.  rows and width multiples of 512.  A measurement aid:
 * no counterpart in the reference. */
enum {
  TK_YS_READ = 0,        /* contiguous read */
  TK_YS_COPY = 1,        /* contiguous a -> b */
  TK_YS_RMW = 2,         /* contiguous in-place update */
  TK_YS_RMW_NT = 3,      /* ... with non-temporal accesses */
  TK_YS_TILE_READ = 4,   /* (tile, 128 columns) per wave, read: the expand kernel's loads */
  TK_YS_TILE_RMW_NT = 5, /* (tile, 128 columns) per wave, in-place update, non-temporal: the expand kernel */
  TK_YS_SHRINK_READ = 6, /* (two tiles, 512 columns) per wave in MFMA operand order: the shrink kernel's loads */
  TK_YS_WALK_READ = 7,   /* one wave walks 16 tiles for 128 columns: the row-contraction kernels' loads */
  TK_YS_LDS_STREAM = 8,  /* 256 blocks of 8 waves load their share of `a` into LDS, 64 KB per step and barrier: the grouped
                            GEMM's operand path with every line from memory (rows * width * 2 a multiple of 16 MiB) */
  TK_YS_LDS_SHARED = 9   /* the same with all blocks walking the first 2 MB, 16 times the steps: every line an L2 hit */
};
int tk_yardstick(int32_t kind, void* a_device, void* b_device, const int32_t* row_of_device, int64_t rows,
                 int32_t width, tk_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TWINKLE_AMD_H */
