// Internal declarations shared by the host C ABI and the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <string>
#include <vector>
#include <map>
#include "../../include/pooled_attn.h"

// ---- kernel-side parameter blocks -------------------------------------------------------------

struct GlueParams {
  const float* q_in; const float* k_in; const float* v_in;   // column-batched f32 inputs
  float* k_out;                                              // in-place k write-back (pa_glue) or nullptr
  const float* qw; const float* kw;                          // norm weights [hd]
  const float* inv_freq;                                     // [n_rot/2] f32, theta^(-2i/n_rot)
  const float2* rope_tab;                                    // [max_seq][n_rot/2] (cos, sin) or nullptr
  float* q_out; float* gate_out;                             // [n_cols][nH*hd]
  uint16_t* k_cache; uint16_t* v_cache;                      // f16 (or int8) [nKV][head_rows][hd] or nullptr
  float* ks_cache; float* vs_cache;                          // int8 caches: scales [nKV][head_rows][hd/32]
  uint32_t head_rows;                                        // rows of one kv head's plane (max_seq + padding)
  uint32_t q_stride, k_stride, v_stride;
  uint32_t n_heads, n_kv_heads, head_dim, n_rot;
  uint32_t base_pos, n_cols;
  uint32_t flags;                                            // PA_FLAG_*; bit 8: rope/norm enabled (0 = pack only)
  float eps;
};

struct AttnParams {
  const float* q; const float* gate;          // f32 [n_cols][stride]
  const uint16_t* k_cache; const uint16_t* v_cache;
  const float* k_scale; const float* v_scale;   // int8 caches: one f32 scale per 32 values, [nKV][head_rows][hd/32]
  float* part_o; float* part_ml;              // split partials: [(col*nH + h)*slots + sp][hd], [..][2]
  void* out;                                  // [n_cols][out_stride]
  uint32_t q_stride, gate_stride, out_stride;
  uint32_t n_heads, n_kv_heads, group;        // group = nH / nKV
  uint32_t base_pos, n_cols;                  // column c sees rows [0, base_pos + c]
  uint32_t split_len, n_splits, slots;
  uint32_t cols_per_group;                    // columns per workgroup (grid z = column groups)
  uint32_t max_seq;
  uint32_t self_row;                          // 1: one-column decode whose own row base_pos is a partial of its own (slot
                                              // = number of splits that hold rows) instead of a streamed row; else 0.
                                              // Its (m, l) sits under every head, its O row under the kv head's first head only
  int out_f16;
  uint32_t direct_out;                        // tile-loop split-K kernel with one split and no own-row partial: the workgroup
                                              // normalises, gates and stores the output itself (no partials, no merge launch)
  float scale;                                // 1 / sqrt(hd)
  uint32_t gate_head_stride;                  // floats between consecutive heads in gate (head_dim, or 2*head_dim
                                              // when gate is read in place from an interleaved [q | gate] column)
  uint32_t part_f16;                          // 1: the O partials in part_o are f16 rows [slot][hd] (single-round decode splits
                                              // merged by the wavefront kernel); 0: f32
  // fused pre-step of pa_attn_decode_step (one column at base_pos; f_q_in == nullptr otherwise): raw projections
  const float* f_q_in; const float* f_k_in; const float* f_v_in;   // [nH][q_head_stride], [nKV][hd], [nKV][hd]
  const float* f_qw; const float* f_kw;       // norm weights [hd] or nullptr
  const float2* rope_tab; const float* inv_freq;
  uint32_t f_q_head_stride, n_rot;
  float eps;
  // gather mode (pa_attn_decode_gather): per column sel[col * sel_stride] = n, then n cache rows; nullptr otherwise
  // sel_max: the longest list the pass was sized for; a longer length word is read as sel_max (the list cannot run
  // into the next column's), a length of 0 gives a column of zeros
  const uint32_t* sel; uint32_t sel_stride, sel_max;
  uint32_t exact_cols;                        // 1: a column-exact verify block in one launch: every column is a column group of its
                                              // own under the plan of a one-column decode (the merge must be the wavefront kernel)
  uint32_t col_groups, ncg_magic, ns_magic;   // tile loop (set by its launcher): the column groups of the pass and ceil(2^32 / d) for d = col_groups
                                              // and d = n_splits, so that the kernel maps its dispatch id to (column group, split, kv head) with
                                              // two multiplies instead of four divisions (0: d is 1, or the ids are too large for the identity)
  uint32_t single_round2;                     // 1: two row blocks on the single-round kernel (splits of one tile per wave)
  uint32_t tile_ilv;                          // tile loop of the split-K kernel on a contiguous cache: rows from one split's first tile
                                              // to the next split's (32 x waves) when the tiles of a kv head are dealt round robin to the
                                              // waves of all its splits; 0 = every split a contiguous range of split_len rows
};

// ---- kernel launchers (defined next to their kernels) ------------------------------------------

// Optional kernel-exact timing of a launch: with both events set the kernel goes out through hipExtLaunchKernelGGL,
// which stamps them with the dispatch's own begin / end timestamps (the clock a kernel trace reports), so
// hipEventElapsedTime(start, stop) is the kernel's duration without launch or event-handling latency.
struct PaTiming { hipEvent_t start = nullptr, stop = nullptr; };
#define PA_LAUNCH(kernel, grid, block, lds, stream, timing, ...)                                                          \
  do {                                                                                                                    \
    if ((timing) && (timing)->start) hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, (timing)->start, (timing)->stop, 0, __VA_ARGS__); \
    else hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                                               \
  } while (0)

hipError_t pa_launch_glue(const GlueParams& p, hipStream_t s);
hipError_t pa_launch_rope_table(float2* tab, const float* inv_freq, uint32_t half, uint32_t n_pos, hipStream_t s);
// waves per workgroup W in {4, 8}; NB = 16-row query blocks per workgroup (1..4); hd in {128, 256}
hipError_t pa_launch_decode(const AttnParams& p, uint32_t hd, uint32_t nb, uint32_t waves, uint32_t col_groups, hipStream_t s, const PaTiming* t = nullptr);
// gather mode: every column attends to its own list of cache rows (p.sel set; cols_per_group == 1, grid z = column)
hipError_t pa_launch_decode_gather(const AttnParams& p, uint32_t hd, hipStream_t s, const PaTiming* t = nullptr);
// the same with the pre-step of the one column fused in (p.f_* set; one 16-row block, n_cols == 1)
hipError_t pa_launch_decode_step(const AttnParams& p, uint32_t hd, hipStream_t s, const PaTiming* t = nullptr);
hipError_t pa_prepare_decode_step(uint32_t hd, bool q8);
hipError_t pa_launch_combine(const AttnParams& p, uint32_t hd, hipStream_t s, const PaTiming* t = nullptr);
// MFMA prefill; returns hipErrorNotSupported for shapes it does not cover
hipError_t pa_launch_prefill(const AttnParams& p, uint32_t hd, uint32_t row_blocks, uint32_t col_groups, hipStream_t s, const PaTiming* t = nullptr);

// one-token projection y = W x (proj_gemv.hip): kind PA_W_*, w = f32 [d_out][d_in] / int8 [d_out][d_in] / nibbles
// [d_out][d_in / 2], scales = f16 bits [d_out][d_in / 32] (quantised kinds); norm_w != nullptr: x is the raw vector and
// the kernel applies rmsnorm with that weight (xn_out != nullptr: also written); acc: y += W x
struct GemvParams {
  const void* w; const uint16_t* scales;
  const float* x; const float* norm_w; float* xn_out; float* y;
  uint32_t d_out, d_in;
  float eps; int acc; int kind;
};
hipError_t pa_launch_gemv(const GemvParams& p, int n_cu, hipStream_t s);

// column-batched projection Y[c][r] = sum_k W[r][k] X[c][k] (proj_gemm.hip): x = f16 bits [n_cols][x_stride], y = f32
// [n_cols][y_stride]; weights as GemvParams; acc: y += W x
struct GemmParams {
  const void* w; const uint16_t* scales;
  const uint16_t* x; float* y;
  uint32_t x_stride, y_stride;
  uint32_t d_out, d_in, n_cols;
  int acc; int kind;
};
hipError_t pa_launch_gemm(const GemmParams& p, int n_cu, hipStream_t s);
// large chunks (proj_gemm_wide.hip): the weights widened once into w16 (f16 in fragment order, the caller's staging), then a
// GEMM over two f16 operands; pa_gemm_wide_serves tells whether a call qualifies
bool pa_gemm_wide_serves(const GemmParams& p, int n_cu);
size_t pa_gemm_wide_staging_bytes(uint32_t d_out, uint32_t d_in);
bool pa_gemm_mid_serves(const GemmParams& p);
hipError_t pa_launch_gemm_wide(const GemmParams& p, uint16_t* w16, bool widen, bool mid, int n_cu, hipStream_t s);
// rmsnorm of n_cols f32 columns, written as f16 (the GEMM's activation operand)
hipError_t pa_launch_rmsnorm_f16(const float* x, uint32_t x_stride, const float* w, uint32_t dim, float eps, uint32_t n_cols,
                                 uint16_t* out, uint32_t out_stride, hipStream_t s);

// int8 caches -> f16 staging cache of the same geometry (glue_kv.hip): rows [0, n_live) widened, [n_live, n_rows) zeroed
hipError_t pa_launch_widen_q8(const void* k8, const void* v8, const float* ks, const float* vs, uint16_t* ko, uint16_t* vo,
                              uint32_t n_kv_heads, uint32_t hd, uint32_t head_rows, uint32_t n_live, uint32_t n_rows, hipStream_t s);

// ---- context -----------------------------------------------------------------------------------

// One layer's caches.  f16 caches: k, v.  int8 caches (PA_FLAG_KV_Q8): k, v hold int8 values (hd bytes a row), ks, vs
// one f32 scale per 32 values.  All head-major [nKV][max_seq + 32][row].
struct pa_layer {
  uint16_t* k = nullptr; uint16_t* v = nullptr; float* ks = nullptr; float* vs = nullptr;
  void* tensor(int which) const { return which == 0 ? (void*)k : which == 1 ? (void*)v : which == 2 ? (void*)ks : (void*)vs; }
};

// A checkpoint slot: per allocated layer a compact head-major copy [nKV][pos][hd] of K and of V rows [0, pos).
struct pa_slot {
  uint32_t pos = 0;
  std::vector<void*> t[4];         // per tensor (K, V, K scales, V scales), indexed by layer; nullptr where absent
};

struct pa_weight {
  int kind = 0;
  uint32_t d_out = 0, d_in = 0;
  void* w = nullptr;              // values plane on the device
  uint16_t* scales = nullptr;     // f16 bits [d_out][d_in / 32]; nullptr for f32 weights
  uint16_t* w16 = nullptr;        // the weights widened to f16 in fragment order, kept from the first large-chunk pa_gemm on
  size_t w16_bytes = 0;           // (while the context's budget lasts); nullptr: widened per call into the context's staging
  hipEvent_t w16_ready = nullptr; // recorded behind the kernel that filled w16, on w16_stream; nullptr once a host wait has seen it
  hipStream_t w16_stream = nullptr;
};

struct pa_ctx {
  pa_config cfg{};
  int device = 0;
  int n_cu = 0;
  hipStream_t own_stream = nullptr;
  hipStream_t stream = nullptr;
  std::vector<pa_layer> layers;
  std::map<uint32_t, pa_slot> slots;
  float* q_buf = nullptr;       // [max_cols][nH*hd]
  float* gate_buf = nullptr;    // [max_cols][nH*hd]
  float* inv_freq = nullptr;    // [n_rot/2]
  float2* rope_tab = nullptr;   // [max_seq][n_rot/2] (cos, sin); nullptr when it would exceed 1 GiB
  float* part_o = nullptr; float* part_ml = nullptr;
  size_t part_o_bytes = 0, part_ml_bytes = 0;
  float* proj_buf = nullptr;    // pa_attn_layer_decode: [q(+gate) | k | v] projections, then attnOut [nH*hd]
  size_t proj_buf_bytes = 0;
  void* w16_buf = nullptr;      // pa_gemm on large chunks: the call's weights widened to f16 [d_out][d_in]
  size_t w16_buf_bytes = 0;
  size_t weight_cache_limit = (size_t)8 << 30, weight_cache_used = 0;   // pa_set_weight_cache: budget of the kept f16 copies
  void* chunk_buf = nullptr;    // pa_attn_layer_prefill: xn f16 [cols][dim], qkv f32 [cols][rows], attnOut f16 [cols][nH*hd]
  size_t chunk_buf_bytes = 0;
  uint16_t* wide_k = nullptr; uint16_t* wide_v = nullptr;   // int8 caches: f16 staging cache of one layer for the prefill kernel
  void* static_scratch = nullptr;   // this device's copy of the library's file-scope scratch array (pa_attn_decode_step_noalloc)
  std::vector<void*> retired;   // outgrown scratch blocks, kept until pa_destroy (a recorded launch may still name them)
  uint32_t decode_splits_override = 0;
  int prefill_tile_mode = 0;    // pa_set_prefill_tile: 0 table, 1 always the matrix-core kernel, 2 never
  // timing
  hipEvent_t t0 = nullptr, t1 = nullptr;
  bool profiling = false;
  std::vector<hipEvent_t> prof_events;   // pairs
  size_t prof_used = 0;
  std::vector<hipEvent_t> prof_aux;      // pairs around the merge launch of a profiled call (stamped, never read; reused in a ring)
  size_t prof_aux_used = 0;
  std::string err;
};
