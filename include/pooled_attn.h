/* pooled_attn.h -- C ABI of the MI355X (gfx950) attention library for pooled's engines.
 *
 * pooled has no FFI on this path: attention is dispatched inline by engine methods that record WebGPU
 * compute passes.  Each entry point below replaces the group of WebGPU dispatches named in its comment
 * (paths relative to the pooled repository).  All functions return PA_OK (0) or a PA_ERR_* code and never
 * abort; pa_last_error() gives the message.  All calls for one context come from one host thread; kernels
 * are enqueued in order on the context's HIP stream and only pa_sync / the host copies block.
 *
 * Pointers named d_* are device (HBM) addresses, h_* are host addresses.  Strides are in elements
 * (floats for f32 buffers), like the FD / FA / MC uniforms of the reference kernels.
 */
#ifndef POOLED_ATTN_H
#define POOLED_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PA_OK 0
#define PA_ERR_INVALID 1      /* bad argument / shape */
#define PA_ERR_UNSUPPORTED 2  /* shape outside the gfx950 table (caller may fall back) */
#define PA_ERR_HIP 3          /* a HIP runtime call failed */
#define PA_ERR_NOMEM 4

/* pa_config.flags */
#define PA_FLAG_QK_NORM 1u    /* per-head RMSNorm of q and k before RoPE (engine/wgsl/base.js:65-79) */
#define PA_FLAG_GATE 2u       /* q input is interleaved [q(hd) | gate(hd)] per head and the output is
                                 multiplied by sigmoid(gate) (engine/wgsl/qwen35.js:370-384, :406-416) */

#define PA_FLAG_KV_Q8 4u      /* int8 caches: values rounded to int8 with one f32 scale per 32 (scale = max|x| / 127),
                                 the reference's kvQ8 mode (kv_store_q8, attn_flash_q8: engine/wgsl/qwen35.js:908-946,
                                 :99-139).  Served by pa_glue_kv / pa_kv_store / pa_attn_decode / pa_attn_prefill /
                                 pa_attn_decode_step / slots and the layer calls; pa_attn_decode_gather returns
                                 PA_ERR_UNSUPPORTED (as the reference: attnDecConfig, engine/wgsl/attn_dec.js:40-41).  A wide
                                 pa_attn_prefill chunk widens the rows it can see into an f16 staging cache the
                                 context allocates on first use (one layer's f16 cache in size) and runs the
                                 matrix-core prefill kernel on it. */

#define PA_FLAG_VERIFY_EXACT 8u /* pa_attn_decode with n_cols > 1 runs every column as the one-column decode at its own position
                                 (its own splits, its own row block): column c then has the bits of pa_attn_decode(base_pos + c,
                                 n_cols = 1), the invariant the reference states for its pair (engine/wgsl/attn_dec.js:12-16,
                                 tests/test_attn_dec.js:89-97) and its speculative decoding leans on (spec greedy == plain
                                 greedy).  Cost: every column streams the K/V rows through its own workgroups; a block whose
                                 columns share one one-column plan runs as one pass in which a split's columns sit side by
                                 side on one L2 (about 2.3x the default block's time), a block that straddles a change of
                                 plan as one pass per column.  Off by default: see the note at pa_attn_decode. */

/* output element types */
#define PA_OUT_F32 0          /* the engine's attnOut feeding wo (engine/qwen35.js:881) */
#define PA_OUT_F16 1

/* Model-shape constants: the fields of the reference's Config and DN uniforms that attention uses
 * (engine/wgsl/base.js:4-9, engine/wgsl/qwen35.js:271-275) plus the engine's sizing inputs
 * (engine/qwen35.js:354-368: maxSeq, batchCols). */
typedef struct pa_config {
  uint32_t n_heads;      /* nH */
  uint32_t n_kv_heads;   /* nKV; nH % nKV == 0, G = nH / nKV */
  uint32_t head_dim;     /* hd: 128 or 256 */
  uint32_t n_rot;        /* rotated dims per head (== head_dim for full RoPE), even */
  float rope_theta;
  float eps;             /* RMSNorm epsilon */
  uint32_t max_seq;      /* cache rows per layer */
  uint32_t n_layers;     /* attention layers (one K and one V cache each) */
  uint32_t max_cols;     /* widest pass (columns) the context must serve */
  uint32_t flags;        /* PA_FLAG_* */
} pa_config;

typedef struct pa_ctx pa_ctx;

/* What the gfx950 table chose for a pass (replaces the reference's load-time calibration and static
 * formulas: engine/autotune.js:10-68, engine/wgsl/attn_dec.js:40-48, engine/wgsl/attn_tile.js:43-56). */
typedef struct pa_plan {
  uint32_t kernel;       /* 0 = split-K decode/verify kernel, 1 = MFMA prefill kernel */
  uint32_t split_len;    /* cache rows per split (split-K kernel with more than 128 rows a split: the rows of a split's
                            32-row tiles, which are dealt round robin to the splits of a kv head, not one contiguous range) */
  uint32_t n_splits;     /* splits over the streamed rows; a one-column decode streams rows 0 .. base_pos - 1 */
  uint32_t col_groups;   /* column groups (workgroups = n_splits x kv heads x col_groups) */
  uint32_t cols_per_group;
  uint32_t waves;        /* wavefronts per workgroup */
  uint32_t row_blocks;   /* 16-row (decode) or 32-row (prefill) query blocks per workgroup */
  uint32_t slots;        /* partial slots per (column, head) the pass needs: n_splits, + 1 for a one-column decode, whose
                            own row base_pos is a partial of its own */
} pa_plan;

/* ---- life cycle (replaces Qwen35Engine / DenseEngine buffer creation, engine/qwen35.js:871-890,
 *      :1102-1104; engine/dense.js:226-227; size check engine/qwen35.js:378-383) ---- */
int pa_create(const pa_config* cfg, pa_ctx** out);
int pa_destroy(pa_ctx* ctx);
/* message of the last failing call on ctx (ctx == NULL: of the last failing pa_create) */
const char* pa_last_error(const pa_ctx* ctx);
/* allocate layer's K and V caches, zero-filled f16.  Device layout (head-major, chosen for the HBM stream of the
 * attention kernels): [n_kv_heads][max_seq + 32][head_dim]; the 32 extra rows per head stay zero. */
int pa_layer_alloc(pa_ctx* ctx, uint32_t layer);
/* use the caller's hipStream_t (NULL: the context's own stream) */
int pa_set_stream(pa_ctx* ctx, void* hip_stream);
int pa_sync(pa_ctx* ctx);

/* ---- device memory helpers for hosts without their own HIP binding (the Node-API addon) ---- */
int pa_malloc(pa_ctx* ctx, size_t bytes, void** d_ptr);
int pa_free(pa_ctx* ctx, void* d_ptr);
int pa_upload(pa_ctx* ctx, void* d_dst, const void* h_src, size_t bytes);     /* blocking */
int pa_download(pa_ctx* ctx, void* h_dst, const void* d_src, size_t bytes);   /* blocking, after queued work */

/* device-to-device copy on the context's stream (not blocking): the engine's slot copies of KV rows are
 * copyBufferToBuffer calls (engine/dense.js:20-47 saveSlot / loadSlot) */
int pa_copy_d2d(pa_ctx* ctx, void* d_dst, const void* d_src, size_t bytes);

/* ---- pre-step ----
 * pa_glue_kv: q de-interleave + QK-RMSNorm + (partial) NeoX RoPE for n_cols columns at positions
 * base_pos + c, and the f16 write of the k and v rows into layer's caches at those positions.
 * Replaces attn_glue_kv (engine/wgsl/layer_fuse.js:87-146), i.e. attn_glue
 * (engine/wgsl/qwen35.js:1082-1136) followed by kv_store (:889-906); for full RoPE shapes it replaces
 * head_norm_dmc + rope_dmc + kv_store_d / attn_glue_d (engine/wgsl/dense.js:144-196, :233-352) with an
 * f16 cache.  Call sites: engine/qwen35.js:1598-1617, :2473-2488; engine/dense.js:394-399.
 *   d_q_in : f32 [n_cols][q_stride]; a column holds [nH][2*hd] (PA_FLAG_GATE) or [nH][hd]
 *   d_k, d_v: f32 [n_cols][k_stride | v_stride], a column holds [nKV][hd]
 *   d_qw, d_kw: f32 [hd] norm weights (ignored without PA_FLAG_QK_NORM)
 * Results: roped q -> the context's q buffer (pa_q_buffer), gate -> pa_gate_buffer, cache rows written. */
int pa_glue_kv(pa_ctx* ctx, uint32_t layer, const float* d_q_in, uint32_t q_stride, const float* d_k,
               uint32_t k_stride, const float* d_v, uint32_t v_stride, const float* d_qw, const float* d_kw,
               uint32_t base_pos, uint32_t n_cols);
/* pa_glue: the same without the cache write; the normed + roped k is written back in place (d_k), as
 * attn_glue does (engine/wgsl/qwen35.js:1082-1136; call site engine/qwen35.js:2473-2483). */
int pa_glue(pa_ctx* ctx, const float* d_q_in, uint32_t q_stride, float* d_k, uint32_t k_stride,
            const float* d_qw, const float* d_kw, uint32_t base_pos, uint32_t n_cols);
/* pa_kv_store: f16 (round-to-nearest-even) write of already-roped k and raw v rows at base_pos + c.
 * Replaces kv_store (engine/wgsl/qwen35.js:889-906; call site engine/qwen35.js:2488). */
int pa_kv_store(pa_ctx* ctx, uint32_t layer, const float* d_k, uint32_t k_stride, const float* d_v,
                uint32_t v_stride, uint32_t base_pos, uint32_t n_cols);
/* the context's q / gate buffers written by pa_glue*: f32 [max_cols][nH*hd] (stride = nH*hd) */
float* pa_q_buffer(pa_ctx* ctx);
float* pa_gate_buffer(pa_ctx* ctx);

/* ---- attention ----
 * pa_attn_decode: split-K flash-decoding for one decode token (n_cols = 1) or a speculative-verify block
 * (n_cols <= max_cols): column c at absolute position base_pos + c attends to cache rows [0, base_pos + c],
 * followed by the log-sum-exp merge and, when d_gate != NULL, the sigmoid gate.
 * Replaces attn_dec + attn_dec_combine(_g) + sigmoid_mul(_mc) (engine/wgsl/attn_dec.js:102-287,
 * engine/wgsl/qwen35.js:406-416, :877-887) and the v1 pair attn_flash + attn_combine(_g)
 * (engine/wgsl/qwen35.js:99-197, :1059-1080, engine/wgsl/layer_fuse.js:148-181).
 * Call sites: engine/qwen35.js:1618-1640 (one token), :2494-2516 (verify columns).
 * A verify column is NOT bit-identical to the one-column decode at the same position unless PA_FLAG_VERIFY_EXACT is set:
 * the columns of a block are stacked into shared matrix-core tiles and the block's splits are chosen from the block,
 * while a one-column decode streams whole 128-row splits and keeps its own row as a separate partial, so the two sum
 * in different orders.  They agree to rounding (the tests bound |block - sequential| by 1e-3; measured 3e-4), which
 * is inside the path's tolerance but weaker than the reference's own guarantee (engine/wgsl/attn_dec.js:12-16): an
 * engine that needs speculative greedy decoding to reproduce plain greedy decoding token for token sets the flag.
 *   d_q   : f32 [n_cols][q_stride], a column holds roped q [nH][hd]; NULL = pa_q_buffer
 *   d_gate: f32 [n_cols][gate_stride] gate pre-activations [nH][hd]; NULL = no gate
 *   d_out : [n_cols][out_stride] of out_dtype, a column holds [nH][hd]
 * pa_attn_prefill: the same contract for a causal prefill chunk of any width: the f16 MFMA kernel, or, for a chunk of
 * few columns (at most one 32- / 64-row block, or a few column groups over a long context, where the K/V stream and
 * not the matrix cores bound the pass), the split-K kernel; pa_plan_query tells which.
 * Replaces attn_flash_tile + attn_combine_tile + sigmoid_mul_mc (engine/wgsl/attn_tile.js:108-193;
 * call site engine/qwen35.js:2489-2493, :2516); one call covers what the reference runs as
 * ceil(n_cols / 16) consecutive 16-column passes (engine/qwen35.js:3843-3860). */
int pa_attn_decode(pa_ctx* ctx, uint32_t layer, const float* d_q, uint32_t q_stride, const float* d_gate,
                   uint32_t gate_stride, uint32_t base_pos, uint32_t n_cols, void* d_out, uint32_t out_stride,
                   int out_dtype);
int pa_attn_prefill(pa_ctx* ctx, uint32_t layer, const float* d_q, uint32_t q_stride, const float* d_gate,
                    uint32_t gate_stride, uint32_t base_pos, uint32_t n_cols, void* d_out, uint32_t out_stride,
                    int out_dtype);
/* pa_attn_decode_step: the whole attention block of one decode token in one call -- pre-step, cache write,
 * split-K attention, merge and gate -- with the pre-step fused into the attention kernel (no separate launch, the
 * roped q never leaves the chip).  Replaces the one-token sequence attn_glue_kv + attn_dec + attn_dec_combine_g
 * (call site engine/qwen35.js:1598-1640; dense: engine/dense.js:394-399 + :463-469) and gives the same cache row
 * bits and the same output as pa_glue_kv followed by pa_attn_decode.
 *   d_q_in: f32 one column [nH][2*hd] (PA_FLAG_GATE: [q | gate] per head) or [nH][hd]
 *   d_k, d_v: f32 [nKV][hd];  d_qw, d_kw: f32 [hd] (ignored without PA_FLAG_QK_NORM)
 *   d_out : [nH][hd] of out_dtype
 * pa_q_buffer / pa_gate_buffer are not written by this call. */
int pa_attn_decode_step(pa_ctx* ctx, uint32_t layer, const float* d_q_in, const float* d_k, const float* d_v,
                        const float* d_qw, const float* d_kw, uint32_t pos, void* d_out, int out_dtype);
/* pa_attn_decode_step_noalloc: pa_attn_decode_step for callers that cannot allocate.  No counterpart in the reference;
 * it exists for callers under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.  Same
 * arguments, same kernels and the same bits as pa_attn_decode_step, but the split partials go to a file-scope device
 * array of the library (8 MiB per GPU, held until the process ends; its device address is looked up at pa_create) and
 * the call makes no hipMalloc / hipFree and creates no events (pa_profile_enable does not see it).  A shape whose
 * partials -- n_heads x (splits + 1) x (head_dim + 2) floats -- do not fit returns PA_ERR_UNSUPPORTED (the MoE shape
 * at 32K uses 4.3 MB).  All calls on one GPU share the array, contexts included: calls that overlap on one GPU (two
 * streams, two contexts) race; calls queued on one stream do not.  Nothing in the array needs clearing between calls:
 * every partial the merge reads is written by the same call. */
int pa_attn_decode_step_noalloc(pa_ctx* ctx, uint32_t layer, const float* d_q_in, const float* d_k, const float* d_v,
                                const float* d_qw, const float* d_kw, uint32_t pos, void* d_out, int out_dtype);
/* pa_attn_decode_gather: decode / verify attention where every column attends to a list of cache rows instead of
 * rows [0, base_pos + c] -- the gather mode of the reference's split-K kernel used by its sparse-attention layers:
 * attn_dec_qsa + attn_dec_qsa_combine(_g) (engine/wgsl/attn_dec.js:33-38, :105, :170-183, :246; dispatch
 * engine/qsa.js:41-56).  Same q / gate / out contract as pa_attn_decode.
 *   d_sel: u32 [n_cols][sel_stride]; column c's list is d_sel[c * sel_stride] = n (0 <= n <= max_rows), then n row
 *          indices < max_seq at d_sel[c * sel_stride + 1 ..], ascending (the reference's QSA_SEL_STRIDE layout).  The
 *          device-side length word is not trusted: n > max_rows is read as max_rows (a list never runs into the next
 *          column's), row indices are clamped to the cache, and n == 0 gives a column of zeros.
 *   max_rows: the longest list of the pass (engine/qsa.js:34 qsaMaxRows); sizes the splits
 * List position t stands where position t stands in pa_attn_decode: with the list 0 .. pos a single column gives
 * pa_attn_decode's result at base_pos = pos to rounding (2e-5; the dense call keeps the column's own row out of the
 * streamed rows, so the two sum in a different order). */
int pa_attn_decode_gather(pa_ctx* ctx, uint32_t layer, const float* d_q, uint32_t q_stride, const float* d_gate,
                          uint32_t gate_stride, const uint32_t* d_sel, uint32_t sel_stride, uint32_t max_rows,
                          uint32_t n_cols, void* d_out, uint32_t out_stride, int out_dtype);
/* which kernel / split / tile shape the table picks (kind: 0 decode/verify, 1 prefill) */
int pa_plan_query(const pa_ctx* ctx, int kind, uint32_t base_pos, uint32_t n_cols, pa_plan* out);
/* override the table's split count for decode passes (0 = table); the reference's attnDecodeSplits
 * option (engine/qwen35.js:266, engine/wgsl/attn_dec.js:42) */
int pa_set_decode_splits(pa_ctx* ctx, uint32_t splits);
/* which kernel serves pa_attn_prefill chunks wider than one split-K row block: 0 = the table's choice (default: the
 * matrix-core kernel, except narrow chunks over long contexts and small chunks, which the split-K kernel serves in
 * column groups), 1 = always the matrix-core kernel, 2 = never (split-K kernel in column groups).  The reference's
 * attnPrefillTile engine option ("auto" / true / false, flippable at run time for A/B runs: engine/qwen35.js:389-401);
 * either kernel's result is within the path's tolerance of the other's. */
int pa_set_prefill_tile(pa_ctx* ctx, int mode);

/* ---- cache access for tests, checkpoints and slot copies (engine/dense.js:20-47 saveSlot/loadSlot
 *      copy rows [0, pos) of each layer) ----  which: 0 = K, 1 = V; the host side is the engine's position-major
 *      view, f16 bits [n_rows][nKV*hd]; the calls translate to and from the device layout and block.
 *      int8 caches: which 0 / 1 are int8 [n_rows][nKV*hd], which 2 / 3 the K / V scales, f32 [n_rows][nKV*hd/32]
 *      (the reference's kCache / vCache / kScale / vScale parts, engine/qwen35.js:121-131) */
int pa_kv_read(pa_ctx* ctx, uint32_t layer, int which, uint32_t row0, uint32_t n_rows, void* h_dst);
int pa_kv_write(pa_ctx* ctx, uint32_t layer, int which, uint32_t row0, uint32_t n_rows, const void* h_src);
/* bytes of one row of the host view of cache tensor `which` (nKV * hd f16 / int8 values, or nKV * hd / 32 f32 scales):
 * what pa_kv_read / pa_kv_write move per row and pa_slot_export / pa_slot_import per saved position -- the part sizes of
 * the reference's saved states (engine/qwen35.js:121-131).  0 for a tensor the context does not have. */
size_t pa_kv_row_bytes(const pa_ctx* ctx, int which);
/* device address of a cache (read-only use; the head-major device layout described at pa_layer_alloc) */
const void* pa_kv_device_ptr(pa_ctx* ctx, uint32_t layer, int which);

/* ---- checkpoint slots: the rows written so far, kept on the device or moved to the host ----
 * Replace the engines' saveSlot / loadSlot / dropSlot (engine/dense.js:20-47, engine/qwen35.js:190-230: a copy of
 * KV rows [0, pos) per layer, made and restored on the GPU queue) and, for the attention layers, the parts of
 * exportSlot / exportState / importState (engine/qwen35.js:121-131, :151-190): per layer one K and one V part of
 * pos * nKV * hd f16, position-major -- the reference's flash-KV part layout, so parts written by either backend
 * load into the other.  slot is a caller-chosen id (the shim maps names to ids).
 * pa_slot_save: device copy of rows [0, pos) of every allocated layer, queued on the context's stream (a slot of the
 *   same id is replaced); pa_slot_load: the copy back, *pos = the saved position; pa_slot_drop frees (unknown id:
 *   no error, as dropSlot); pa_slot_pos: the saved position.
 * pa_slot_create + pa_slot_import build a slot from host parts (then pa_slot_load restores it);
 * pa_slot_export reads one part back.  Host copies block. */
int pa_slot_save(pa_ctx* ctx, uint32_t slot, uint32_t pos);
int pa_slot_load(pa_ctx* ctx, uint32_t slot, uint32_t* pos);
int pa_slot_drop(pa_ctx* ctx, uint32_t slot);
int pa_slot_pos(pa_ctx* ctx, uint32_t slot, uint32_t* pos);
int pa_slot_create(pa_ctx* ctx, uint32_t slot, uint32_t pos);
int pa_slot_export(pa_ctx* ctx, uint32_t slot, uint32_t layer, int which, void* h_dst);
int pa_slot_import(pa_ctx* ctx, uint32_t slot, uint32_t layer, int which, const void* h_src);

/* ---- timing on the context's stream (HIP events; replaces the reference's timestamp-query passes,
 *      tests/prof/gpuprof.js:1-16) ----
 * pa_timer_start / pa_timer_stop bracket a region; stop blocks and returns milliseconds.
 * pa_profile_enable(1) additionally times every attention call's main kernel (the split-K or prefill kernel, not
 * glue / merge) with an event pair stamped by the dispatch itself (the kernel's own begin / end timestamps, the
 * figure a kernel trace reports; the call's merge launch is stamped too, unread, because a kernel between unstamped
 * neighbours reads about a microsecond longer than in a trace, where every dispatch is stamped); pa_profile_read blocks, returns the sum of those durations and their count
 * since the last read, and resets them.  pa_profile_read_each does the same but hands back every launch's own
 * duration, in launch order (ms[0 .. min(*count, cap))); *count is the number of launches timed since the last read),
 * so that a caller can report a median instead of a mean. */
int pa_timer_start(pa_ctx* ctx);
int pa_timer_stop(pa_ctx* ctx, float* ms);
int pa_profile_enable(pa_ctx* ctx, int on);
int pa_profile_read(pa_ctx* ctx, float* ms_sum, uint32_t* count);
int pa_profile_read_each(pa_ctx* ctx, float* ms, uint32_t cap, uint32_t* count);

/* ---- projections either side of the attention block, one-token passes.  Replace the reference's matvec /
 *      matvec_q8 / matvec_q4 dispatches and their cooperative, accumulating and normed forms
 *      (engine/wgsl/base.js:15-118, engine/wgsl/coop.js:236-420); built by the engine's mv() / mvN() helpers
 *      (engine/qwen35.js:906-922) and recorded around the attention block at engine/qwen35.js:1591-1597 and :1641.
 *      Weight kinds are the reference's split planes (engine/qwen35.js:894-903): ---- */
#define PA_W_F32 0    /* f32 [d_out][d_in] row-major (engine/wgsl/base.js:15-30) */
#define PA_W_Q8_0 1   /* int8 [d_out][d_in] + one f16 scale per 32 values, [d_out][d_in / 32] (base.js:32-63) */
#define PA_W_Q4_0 2   /* nibbles [d_out][d_in / 2]: byte j of a block's 16 = element j (low) and j + 16 (high), value =
                         nibble - 8; scales as Q8_0 (base.js:81-118) */
typedef struct pa_weight pa_weight;
/* copies a weight matrix to the device.  h_w: the values plane (f32 / int8 / packed nibbles), h_scales: f16 bits
 * (NULL for PA_W_F32).  d_in must be a multiple of 32 and at most 8192.  A handle belongs to the
 * context that made it: use and destroy it through that context only (pa_gemm may attach a derived copy to it, see
 * pa_set_weight_cache, on that context's stream). */
int pa_weight_create(pa_ctx* ctx, int kind, uint32_t d_out, uint32_t d_in, const void* h_w, const void* h_scales, pa_weight** out);
int pa_weight_destroy(pa_ctx* ctx, pa_weight* w);
/* y[d_out] = W x[d_in]; acc != 0: y += W x (matvec*_coop_acc: the residual add folded into the GEMV) */
int pa_gemv(pa_ctx* ctx, const pa_weight* w, const float* d_x, float* d_y, int acc);
/* y = W rmsnorm(x_raw) with xn = (x * inv) * norm_w, inv = 1 / sqrt(mean(x^2) + eps), eps from pa_config
 * (matvec*_coop_n; rmsnorm: engine/wgsl/base.js:119-152).  d_xn_out != NULL: xn is also written there, as
 * workgroup 0 of the reference's kernel does for the layer's later dispatches. */
int pa_gemv_norm(pa_ctx* ctx, const pa_weight* w, const float* d_x_raw, const float* d_norm_w, float* d_xn_out, float* d_y);
/* One token through the attention half of a full-attention layer, as _encodeLayerR records it
 * (engine/qwen35.js:1586-1641): input rmsnorm -> [q | k | v] projections -> pre-step + cache write -> split-K
 * attention -> merge + gate -> output projection accumulated into the residual.  w_qkv: rows [q (n_heads x head_dim,
 * x 2 with PA_FLAG_GATE: q | gate interleaved per head) | k | v] x dim, one fused weight (the reference fuses k | v,
 * engine/qwen35.js:1109-1114); w_o: dim x (n_heads x head_dim).  d_x [dim] is read and updated in place.  Four
 * launches: normed GEMV, fused decode step (2), accumulating GEMV.  f16 or int8 caches. */
int pa_attn_layer_decode(pa_ctx* ctx, uint32_t layer, const pa_weight* w_qkv, const pa_weight* w_o, const float* d_attn_norm_w,
                         const float* d_qw, const float* d_kw, float* d_x, uint32_t pos);

/* ---- the same projections for column-batched passes (prefill chunks, verify blocks) on the f16 matrix cores.
 *      Replace the reference's batched GEMMs over the same weight planes (engine/wgsl/gemm.js, gemm_sgm.js,
 *      gemm_wide.js; dispatched at engine/qwen35.js:2142-2170, :2600-2620) with its "f16" prefill math
 *      (gemm.js:31-36): dequantised weights and activations rounded to f16, products and sums f32. ---- */
/* xn[c] = f16(rmsnorm(x[c]) * norm_w) for n_cols columns of dim floats (strides in elements); eps from pa_config */
int pa_rmsnorm_f16(pa_ctx* ctx, const float* d_x, uint32_t x_stride, const float* d_norm_w, uint32_t dim, uint32_t n_cols,
                   void* d_xn_f16, uint32_t xn_stride);
/* y[c][0 .. d_out) = W x[c] for n_cols columns; x: f16 bits, stride in f16 elements (>= d_in, multiple of 8);
 * y: f32, stride in floats; acc != 0: y += W x.  Chunks of up to 16 columns (verify blocks, the reference's 16-column
 * passes through its batched matvec, engine/wgsl/coop.js) are served by a kernel that streams the packed weights
 * once per launch; wider chunks run on the matrix cores; same operand precision either way. */
int pa_gemm(pa_ctx* ctx, const pa_weight* w, const void* d_x_f16, uint32_t x_stride, uint32_t n_cols, float* d_y, uint32_t y_stride, int acc);
/* Chunks of more than 16 columns (over d_in a multiple of 128) run on GEMMs over two f16 operands: the weight handle's values widened to f16
 * ((nibble - 8) * scale, int8 * scale, f32 rounded -- the arithmetic of the tiled kernel's staging, so results do not
 * depend on which way a call goes) in matrix-core fragment order.  That copy (2 bytes a weight) is made on the first
 * such call on a handle (which therefore allocates: not under stream capture) and kept until pa_weight_destroy, while
 * the copies kept by this context stay within max_bytes (default 8 GiB; 0: keep none); past the budget a call widens
 * into per-context staging every time (+8 % on a 4096 x 9216 x 2048 chunk, about +10 us on a 64-column one).  Changing the budget keeps what is
 * already held.  No counterpart in the reference, whose WGSL GEMMs dequantise in the inner loop. */
int pa_set_weight_cache(pa_ctx* ctx, size_t max_bytes);
/* n_cols tokens at positions base_pos .. through the attention half of a full-attention layer, as
 * _encodeLayerBatch / _encodeLayerWide record it (engine/qwen35.js:2416-2425, :2827): rmsnorm -> [q | k | v] GEMM ->
 * pre-step + cache write -> causal attention -> gate -> wo GEMM accumulated into the residual columns d_x
 * [n_cols][x_stride] (f32, read and updated in place).  Weights as pa_attn_layer_decode.  Five launches (six when
 * the attention pass is split).  n_cols <= max_cols.  On int8 caches one more launch widens the visible rows for the
 * prefill kernel (as pa_attn_prefill on such caches). */
int pa_attn_layer_prefill(pa_ctx* ctx, uint32_t layer, const pa_weight* w_qkv, const pa_weight* w_o, const float* d_attn_norm_w,
                          const float* d_qw, const float* d_kw, float* d_x, uint32_t x_stride, uint32_t base_pos, uint32_t n_cols);

/* library / device description, e.g. "pooled_attn 0.1 gfx950 256CU" (storage owned by the library, one buffer per
 * calling thread) */
const char* pa_version(void);

#ifdef __cplusplus
}
#endif
#endif
