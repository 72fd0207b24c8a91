// Host side of the C ABI (include/pooled_attn.h): context, caches, the gfx950 plan table, launches.
#include "pa_internal.h"
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>

static thread_local std::string g_create_err;

// Scratch of the allocation-free entry point pa_attn_decode_step_noalloc: the split partials of one decode token live
// in this file-scope device array instead of a buffer the context allocates.  Every GPU the library runs on holds
// its own copy until the process ends.  Host code never uses the array's name as an address: pa_create looks the
// device address up once per device (hipGetSymbolAddress with that device current) and everything -- kernel
// arguments included -- goes through that pointer.
#define PA_STATIC_SCRATCH_BYTES (8u << 20)
#define PA_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[PA_STATIC_SCRATCH_BYTES];
static void* g_scratch_ptr[PA_MAX_DEVICES];
static std::mutex g_scratch_mutex;

static int fail(pa_ctx* ctx, int code, const std::string& msg) {
  if (ctx) ctx->err = msg; else g_create_err = msg;
  return code;
}
static int fail_hip(pa_ctx* ctx, hipError_t e, const char* what) {
  return fail(ctx, e == hipErrorOutOfMemory ? PA_ERR_NOMEM : PA_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
}
#define HIPCHK(ctx, call) do { hipError_t e_ = (call); if (e_ != hipSuccess) return fail_hip(ctx, e_, #call); } while (0)

static inline uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }
static int ensure_partials(pa_ctx* ctx, uint32_t n_cols, uint32_t slots);

extern "C" const char* pa_version(void) {
  static thread_local char buf[128];
  int dev = 0, cus = 0;
  hipDeviceProp_t pr;
  if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&pr, dev) == hipSuccess) {
    cus = pr.multiProcessorCount;
    snprintf(buf, sizeof buf, "pooled_attn 0.1 %s %dCU", pr.gcnArchName, cus);
  } else {
    snprintf(buf, sizeof buf, "pooled_attn 0.1 (no HIP device)");
  }
  return buf;
}

extern "C" const char* pa_last_error(const pa_ctx* ctx) { return ctx ? ctx->err.c_str() : g_create_err.c_str(); }

extern "C" int pa_create(const pa_config* cfg, pa_ctx** out) {
  if (!cfg || !out) return fail(nullptr, PA_ERR_INVALID, "pa_create: null argument");
  *out = nullptr;
  const pa_config& c = *cfg;
  if (c.n_heads == 0 || c.n_kv_heads == 0 || c.n_heads % c.n_kv_heads != 0)
    return fail(nullptr, PA_ERR_INVALID, "pa_create: n_heads must be a positive multiple of n_kv_heads");
  if (c.head_dim != 128 && c.head_dim != 256)
    return fail(nullptr, PA_ERR_UNSUPPORTED, "pa_create: head_dim must be 128 or 256 on the gfx950 table");
  if (c.n_heads / c.n_kv_heads > (c.head_dim == 256 ? 32u : 64u))
    return fail(nullptr, PA_ERR_UNSUPPORTED, "pa_create: too many query heads per kv head for the gfx950 table");
  if (c.n_rot == 0 || (c.n_rot & 1) || c.n_rot > c.head_dim)
    return fail(nullptr, PA_ERR_INVALID, "pa_create: n_rot must be even and in (0, head_dim]");
  if (c.max_seq == 0 || c.n_layers == 0 || c.max_cols == 0 || c.max_cols > 65535)
    return fail(nullptr, PA_ERR_INVALID, "pa_create: max_seq, n_layers, max_cols must be positive (max_cols <= 65535)");
  if (!(c.rope_theta > 0.f) || !(c.eps >= 0.f))
    return fail(nullptr, PA_ERR_INVALID, "pa_create: rope_theta must be > 0 and eps >= 0");
  int ndev = 0;
  hipError_t e = hipGetDeviceCount(&ndev);
  if (e != hipSuccess || ndev == 0) return fail(nullptr, PA_ERR_HIP, "pa_create: no HIP device");
  pa_ctx* ctx = new (std::nothrow) pa_ctx();
  if (!ctx) return fail(nullptr, PA_ERR_NOMEM, "pa_create: out of host memory");
  ctx->cfg = c;
  ctx->layers.resize(c.n_layers);
  hipDeviceProp_t pr;
  if ((e = hipGetDevice(&ctx->device)) != hipSuccess || (e = hipGetDeviceProperties(&pr, ctx->device)) != hipSuccess) {
    delete ctx; return fail_hip(nullptr, e, "pa_create: device query");
  }
  if (strncmp(pr.gcnArchName, "gfx950", 6) != 0) {
    std::string m = std::string("pa_create: built for gfx950, device is ") + pr.gcnArchName;
    delete ctx; return fail(nullptr, PA_ERR_UNSUPPORTED, m);
  }
  ctx->n_cu = pr.multiProcessorCount;
  if (ctx->device < 0 || ctx->device >= PA_MAX_DEVICES) { delete ctx; return fail(nullptr, PA_ERR_UNSUPPORTED, "pa_create: device ordinal beyond the library's table"); }
  {
    // this device's address of the static scratch array (the device is current: hipGetDevice above)
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[ctx->device]) {
      void* ptr = nullptr;
      if ((e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))) != hipSuccess || !ptr) { delete ctx; return fail_hip(nullptr, e, "pa_create: hipGetSymbolAddress(scratch)"); }
      g_scratch_ptr[ctx->device] = ptr;
    }
    ctx->static_scratch = g_scratch_ptr[ctx->device];
  }
  if ((e = pa_prepare_decode_step(c.head_dim, (c.flags & PA_FLAG_KV_Q8) != 0)) != hipSuccess) { delete ctx; return fail_hip(nullptr, e, "pa_create: kernel set-up"); }
  const size_t qbytes = (size_t)c.max_cols * c.n_heads * c.head_dim * sizeof(float);
  std::vector<float> freq(c.n_rot / 2);
  for (uint32_t i = 0; i < c.n_rot / 2; i++) freq[i] = (float)std::pow((double)c.rope_theta, -(2.0 * i) / (double)c.n_rot);
  bool ok = (e = hipStreamCreateWithFlags(&ctx->own_stream, hipStreamNonBlocking)) == hipSuccess
         && (e = hipMalloc((void**)&ctx->q_buf, qbytes)) == hipSuccess
         && (e = hipMalloc((void**)&ctx->gate_buf, qbytes)) == hipSuccess
         && (e = hipMalloc((void**)&ctx->inv_freq, freq.size() * sizeof(float))) == hipSuccess
         && (e = hipMemcpy(ctx->inv_freq, freq.data(), freq.size() * sizeof(float), hipMemcpyHostToDevice)) == hipSuccess
         && (e = hipEventCreate(&ctx->t0)) == hipSuccess && (e = hipEventCreate(&ctx->t1)) == hipSuccess;
  if (!ok) { int rc = fail_hip(nullptr, e, "pa_create: allocation"); pa_destroy(ctx); return rc; }
  ctx->stream = ctx->own_stream;
  // (cos, sin) of every (position, rotated pair), built once: the pre-step then loads 8 bytes instead of
  // evaluating an f64 sincos per pair.  Contexts whose table would pass 1 GiB evaluate in the kernel.
  const size_t tab_bytes = (size_t)c.max_seq * (c.n_rot / 2) * sizeof(float2);
  if (tab_bytes <= ((size_t)1 << 30)) {
    ok = (e = hipMalloc((void**)&ctx->rope_tab, tab_bytes)) == hipSuccess
      && (e = pa_launch_rope_table(ctx->rope_tab, ctx->inv_freq, c.n_rot / 2, c.max_seq, ctx->stream)) == hipSuccess
      && (e = hipStreamSynchronize(ctx->stream)) == hipSuccess;
    if (!ok) { int rc = fail_hip(nullptr, e, "pa_create: rope table"); pa_destroy(ctx); return rc; }
  }
  // split partials for a one-column decode at any position: at most two workgroup slots a CU and the column's own row
  // (wider passes and split overrides grow the buffers on first use)
  {
    const uint32_t slots = 2u * (uint32_t)ctx->n_cu / c.n_kv_heads + 2;
    int rc = ensure_partials(ctx, 1, slots);
    if (rc) { g_create_err = ctx->err; pa_destroy(ctx); return rc; }
  }
  *out = ctx;
  return PA_OK;
}

static void slot_free(pa_slot& sl);

// caches: tensors per layer (K, V [, K scales, V scales]) and the bytes of one kv head's row of each
static inline bool kv_q8(const pa_ctx* ctx) { return (ctx->cfg.flags & PA_FLAG_KV_Q8) != 0; }
static inline int n_tensors(const pa_ctx* ctx) { return kv_q8(ctx) ? 4 : 2; }
static inline size_t head_row_bytes(const pa_ctx* ctx, int which) {
  const size_t hd = ctx->cfg.head_dim;
  return which >= 2 ? hd / 32 * sizeof(float) : (kv_q8(ctx) ? hd : hd * 2);
}


extern "C" int pa_destroy(pa_ctx* ctx) {
  if (!ctx) return PA_OK;
  if (ctx->own_stream) (void)hipStreamSynchronize(ctx->own_stream);
  for (auto& L : ctx->layers) for (int w = 0; w < 4; w++) if (L.tensor(w)) (void)hipFree(L.tensor(w));
  for (auto& kv : ctx->slots) slot_free(kv.second);
  if (ctx->q_buf) (void)hipFree(ctx->q_buf);
  if (ctx->gate_buf) (void)hipFree(ctx->gate_buf);
  if (ctx->inv_freq) (void)hipFree(ctx->inv_freq);
  if (ctx->rope_tab) (void)hipFree(ctx->rope_tab);
  if (ctx->part_o) (void)hipFree(ctx->part_o);
  if (ctx->part_ml) (void)hipFree(ctx->part_ml);
  if (ctx->proj_buf) (void)hipFree(ctx->proj_buf);
  if (ctx->chunk_buf) (void)hipFree(ctx->chunk_buf);
  if (ctx->w16_buf) (void)hipFree(ctx->w16_buf);
  if (ctx->wide_k) (void)hipFree(ctx->wide_k);
  if (ctx->wide_v) (void)hipFree(ctx->wide_v);
  for (void* r : ctx->retired) (void)hipFree(r);
  for (auto ev : ctx->prof_events) (void)hipEventDestroy(ev);
  for (auto ev : ctx->prof_aux) (void)hipEventDestroy(ev);
  if (ctx->t0) (void)hipEventDestroy(ctx->t0);
  if (ctx->t1) (void)hipEventDestroy(ctx->t1);
  if (ctx->own_stream) (void)hipStreamDestroy(ctx->own_stream);
  delete ctx;
  return PA_OK;
}

extern "C" int pa_layer_alloc(pa_ctx* ctx, uint32_t layer) {
  if (!ctx) return PA_ERR_INVALID;
  if (layer >= ctx->cfg.n_layers) return fail(ctx, PA_ERR_INVALID, "pa_layer_alloc: layer out of range");
  pa_layer& L = ctx->layers[layer];
  if (L.k) return PA_OK;
  // head-major, 32 rows of zero padding after each kv head's max_seq rows: the attention kernels load whole
  // 32-row tiles unconditionally
  void* t[4] = {nullptr, nullptr, nullptr, nullptr};
  for (int w = 0; w < n_tensors(ctx); w++) {
    const size_t bytes = ((size_t)ctx->cfg.max_seq + 32) * ctx->cfg.n_kv_heads * head_row_bytes(ctx, w);
    hipError_t e = hipMalloc(&t[w], bytes);
    if (e == hipSuccess) e = hipMemsetAsync(t[w], 0, bytes, ctx->stream);
    if (e != hipSuccess) { for (int x = 0; x < 4; x++) if (t[x]) (void)hipFree(t[x]); return fail_hip(ctx, e, "pa_layer_alloc: cache allocation"); }
  }
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  L.k = (uint16_t*)t[0]; L.v = (uint16_t*)t[1]; L.ks = (float*)t[2]; L.vs = (float*)t[3];
  return PA_OK;
}

extern "C" int pa_set_stream(pa_ctx* ctx, void* hip_stream) {
  if (!ctx) return PA_ERR_INVALID;
  ctx->stream = hip_stream ? (hipStream_t)hip_stream : ctx->own_stream;
  return PA_OK;
}
extern "C" int pa_sync(pa_ctx* ctx) {
  if (!ctx) return PA_ERR_INVALID;
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return PA_OK;
}

extern "C" int pa_malloc(pa_ctx* ctx, size_t bytes, void** d_ptr) {
  if (!ctx || !d_ptr) return PA_ERR_INVALID;
  *d_ptr = nullptr;
  HIPCHK(ctx, hipMalloc(d_ptr, bytes ? bytes : 16));
  return PA_OK;
}
extern "C" int pa_free(pa_ctx* ctx, void* d_ptr) {
  if (!ctx) return PA_ERR_INVALID;
  if (d_ptr) { HIPCHK(ctx, hipStreamSynchronize(ctx->stream)); HIPCHK(ctx, hipFree(d_ptr)); }
  return PA_OK;
}
extern "C" int pa_upload(pa_ctx* ctx, void* d_dst, const void* h_src, size_t bytes) {
  if (!ctx || (!d_dst && bytes) || (!h_src && bytes)) return PA_ERR_INVALID;
  if (!bytes) return PA_OK;
  HIPCHK(ctx, hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return PA_OK;
}
extern "C" int pa_download(pa_ctx* ctx, void* h_dst, const void* d_src, size_t bytes) {
  if (!ctx || (!h_dst && bytes) || (!d_src && bytes)) return PA_ERR_INVALID;
  if (!bytes) return PA_OK;
  HIPCHK(ctx, hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  return PA_OK;
}

extern "C" int pa_copy_d2d(pa_ctx* ctx, void* d_dst, const void* d_src, size_t bytes) {
  if (!ctx || (!d_dst && bytes) || (!d_src && bytes)) return PA_ERR_INVALID;
  if (!bytes) return PA_OK;
  HIPCHK(ctx, hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
  return PA_OK;
}

extern "C" float* pa_q_buffer(pa_ctx* ctx) { return ctx ? ctx->q_buf : nullptr; }
extern "C" float* pa_gate_buffer(pa_ctx* ctx) { return ctx ? ctx->gate_buf : nullptr; }

// ---- pre-step ----------------------------------------------------------------------------------

static int check_cols(pa_ctx* ctx, const char* who, uint32_t layer, bool need_layer, uint32_t base_pos, uint32_t n_cols) {
  if (n_cols == 0 || n_cols > ctx->cfg.max_cols) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": n_cols must be in [1, max_cols]");
  if ((uint64_t)base_pos + n_cols > ctx->cfg.max_seq) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": base_pos + n_cols exceeds max_seq");
  if (need_layer) {
    if (layer >= ctx->cfg.n_layers) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": layer out of range");
    if (!ctx->layers[layer].k) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": layer has no cache (call pa_layer_alloc)");
  }
  return PA_OK;
}

static void fill_glue(const pa_ctx* ctx, GlueParams& p) {
  const pa_config& c = ctx->cfg;
  memset(&p, 0, sizeof p);
  p.inv_freq = ctx->inv_freq; p.rope_tab = ctx->rope_tab;
  p.q_out = ctx->q_buf; p.gate_out = ctx->gate_buf;
  p.n_heads = c.n_heads; p.n_kv_heads = c.n_kv_heads; p.head_dim = c.head_dim; p.n_rot = c.n_rot;
  p.flags = c.flags | 0x100u;
  p.eps = c.eps;
  p.head_rows = c.max_seq + 32;
}

extern "C" int pa_glue_kv(pa_ctx* ctx, uint32_t layer, const float* d_q_in, uint32_t q_stride, const float* d_k,
                          uint32_t k_stride, const float* d_v, uint32_t v_stride, const float* d_qw, const float* d_kw,
                          uint32_t base_pos, uint32_t n_cols) {
  if (!ctx) return PA_ERR_INVALID;
  int rc = check_cols(ctx, "pa_glue_kv", layer, true, base_pos, n_cols);
  if (rc) return rc;
  const pa_config& c = ctx->cfg;
  const uint32_t qcol = c.n_heads * c.head_dim * ((c.flags & PA_FLAG_GATE) ? 2 : 1), kvd = c.n_kv_heads * c.head_dim;
  if (!d_q_in || !d_k || !d_v) return fail(ctx, PA_ERR_INVALID, "pa_glue_kv: null input");
  if ((c.flags & PA_FLAG_QK_NORM) && (!d_qw || !d_kw)) return fail(ctx, PA_ERR_INVALID, "pa_glue_kv: norm weights required");
  if (q_stride < qcol || k_stride < kvd || v_stride < kvd) return fail(ctx, PA_ERR_INVALID, "pa_glue_kv: column stride shorter than a column");
  GlueParams p; fill_glue(ctx, p);
  p.q_in = d_q_in; p.k_in = d_k; p.v_in = d_v; p.qw = d_qw; p.kw = d_kw;
  p.k_cache = ctx->layers[layer].k; p.v_cache = ctx->layers[layer].v; p.ks_cache = ctx->layers[layer].ks; p.vs_cache = ctx->layers[layer].vs;
  p.q_stride = q_stride; p.k_stride = k_stride; p.v_stride = v_stride;
  p.base_pos = base_pos; p.n_cols = n_cols;
  HIPCHK(ctx, pa_launch_glue(p, ctx->stream));
  return PA_OK;
}

extern "C" int pa_glue(pa_ctx* ctx, const float* d_q_in, uint32_t q_stride, float* d_k, uint32_t k_stride,
                       const float* d_qw, const float* d_kw, uint32_t base_pos, uint32_t n_cols) {
  if (!ctx) return PA_ERR_INVALID;
  int rc = check_cols(ctx, "pa_glue", 0, false, base_pos, n_cols);
  if (rc) return rc;
  const pa_config& c = ctx->cfg;
  const uint32_t qcol = c.n_heads * c.head_dim * ((c.flags & PA_FLAG_GATE) ? 2 : 1), kvd = c.n_kv_heads * c.head_dim;
  if (!d_q_in || !d_k) return fail(ctx, PA_ERR_INVALID, "pa_glue: null input");
  if ((c.flags & PA_FLAG_QK_NORM) && (!d_qw || !d_kw)) return fail(ctx, PA_ERR_INVALID, "pa_glue: norm weights required");
  if (q_stride < qcol || k_stride < kvd) return fail(ctx, PA_ERR_INVALID, "pa_glue: column stride shorter than a column");
  GlueParams p; fill_glue(ctx, p);
  p.q_in = d_q_in; p.k_in = d_k; p.k_out = d_k; p.qw = d_qw; p.kw = d_kw;
  p.q_stride = q_stride; p.k_stride = k_stride;
  p.base_pos = base_pos; p.n_cols = n_cols;
  HIPCHK(ctx, pa_launch_glue(p, ctx->stream));
  return PA_OK;
}

extern "C" int pa_kv_store(pa_ctx* ctx, uint32_t layer, const float* d_k, uint32_t k_stride, const float* d_v,
                           uint32_t v_stride, uint32_t base_pos, uint32_t n_cols) {
  if (!ctx) return PA_ERR_INVALID;
  int rc = check_cols(ctx, "pa_kv_store", layer, true, base_pos, n_cols);
  if (rc) return rc;
  const pa_config& c = ctx->cfg;
  const uint32_t kvd = c.n_kv_heads * c.head_dim;
  if (!d_k || !d_v) return fail(ctx, PA_ERR_INVALID, "pa_kv_store: null input");
  if (k_stride < kvd || v_stride < kvd) return fail(ctx, PA_ERR_INVALID, "pa_kv_store: column stride shorter than a column");
  GlueParams p; fill_glue(ctx, p);
  p.n_heads = 0;            // key heads only
  p.flags = 0;              // pack only: no norm, no rope
  p.k_in = d_k; p.v_in = d_v;
  p.k_cache = ctx->layers[layer].k; p.v_cache = ctx->layers[layer].v; p.ks_cache = ctx->layers[layer].ks; p.vs_cache = ctx->layers[layer].vs;
  p.k_stride = k_stride; p.v_stride = v_stride;
  p.base_pos = base_pos; p.n_cols = n_cols;
  HIPCHK(ctx, pa_launch_glue(p, ctx->stream));
  return PA_OK;
}

// ---- the gfx950 plan table ----------------------------------------------------------------------
// Decode / verify (split-K kernel): a workgroup is 4 wavefronts, each streaming 32-position tiles of one
// kv head; rows = columns x G stacked into 16-row MFMA blocks (at most 4 per workgroup, more columns go to
// further column groups).  One 16-row block over a context that two workgroups a CU hold as one tile per wave runs
// on the single-round kernel; everything longer or wider on the tile loop, split so that one workgroup lands on each
// CU (down to one tile per wave on short contexts).
// self_ok: a one-column decode keeps the column's own row out of the streamed rows (the kernel turns it
// into one more partial: slots = n_splits + 1), so a token at a multiple of the split length streams whole tiles only.
static bool plan_self_row(const pa_plan& pl) { return pl.kernel == 0 && pl.slots == pl.n_splits + 1; }
// f16 O partials: the single-round split-K kernel (one row block, one tile per wave) merged by the wavefront kernel
// (pa_launch_combine takes the other merge kernel from 16 columns on), from 64 splits on: each partial's rounding
// (2^-12 of a 128-row average of V) then enters the output with a weight of a sixty-fourth or less, an order of
// magnitude under what the f16 probabilities of the MFMA path already cost; shorter contexts, where a partial IS most
// of the output, and every other pass keep f32 partials.
// round-robin tiles: the tile loop of the split-K kernel (every plan of that kernel but the single-round one) with more
// than one split; the value is the distance between the first rows of two splits
// two row blocks on the single-round kernel: what plan_decode picks when a verify block's context fits
// one round of one-tile-per-wave splits at one workgroup a CU (a pass of a single split stays on the tile loop)
static bool plan_single_round2(const pa_plan& pl) {
  return pl.kernel == 0 && pl.row_blocks == 2 && pl.waves == 4 && pl.split_len == 32 * pl.waves && pl.n_splits > 1;
}
static uint32_t plan_tile_ilv(const pa_plan& pl) {
  return pl.kernel == 0 && pl.split_len != 32 * pl.waves && pl.n_splits > 1 ? 32 * pl.waves : 0;
}
#define PA_F16_PARTIALS_MIN_SPLITS 64u
static bool plan_f16_partials(const pa_plan& pl, uint32_t n_cols) {
  return pl.kernel == 0 && pl.row_blocks == 1 && pl.split_len == 32 * pl.waves && n_cols < 16 && pl.n_splits >= PA_F16_PARTIALS_MIN_SPLITS;
}
// rows_cap (optional): at most this many stacked rows per workgroup (16 or 32) instead of the table's choice;
// one_split: the whole context as one split per workgroup -- with no own-row partial the kernel then writes the
// output itself (no partials, no merge launch).  Both are what plan_prefill asks for on small chunks.
static int plan_decode(const pa_ctx* ctx, uint32_t base_pos, uint32_t n_cols, pa_plan* pl, bool self_ok = true,
                       uint32_t rows_cap = 0, bool one_split = false) {
  const pa_config& c = ctx->cfg;
  const uint32_t G = c.n_heads / c.n_kv_heads;
  // rows per workgroup: 16-row blocks whose O^T accumulators fit the register file next to the
  // in-flight K/V tile (hd 256: 2 blocks, 3 in the case below; hd 128: 4 blocks)
  // hd 256: three blocks (48 rows) when that saves a column group and the context is long enough to fill the chip
  // with splits of six tiles a wave (27B shape, 8 columns at 64K: one group of 48 rows instead of two)
  uint32_t max_rows = c.head_dim == 256 ? 32 : 64;
  if (c.head_dim == 256 && n_cols * G > 32 && 48 / G > 0) {
    const uint32_t g32 = ceil_div(n_cols, 32 / G), g48 = ceil_div(n_cols, 48 / G);
    const uint32_t splits48 = ceil_div(base_pos + n_cols, 32) / (6 * 4);
    if (g48 < g32 && !ctx->decode_splits_override && (uint64_t)splits48 * c.n_kv_heads * g48 >= (uint64_t)ctx->n_cu) max_rows = 48;
  }
  if (rows_cap) max_rows = rows_cap;
  uint32_t cw = n_cols, groups = 1;
  if (n_cols * G > max_rows) { cw = max_rows / G; if (cw == 0) return PA_ERR_UNSUPPORTED; groups = ceil_div(n_cols, cw); }
  uint32_t nb = ceil_div(cw * G, 16);
  // one-launch small chunks at head_dim 128 and two row blocks, at most one workgroup a CU: eight waves (see
  // pa_launch_decode).  Measured: 512 columns at 1536 (256 workgroups) 24.5 -> 22.2 us; 1024 columns from 0 (512
  // workgroups, which four waves run two a CU) 20.3 -> 23.9 us, hence the bound.
  const uint32_t W = one_split && c.head_dim == 128 && nb == 2 && !kv_q8(ctx) && (uint64_t)groups * c.n_kv_heads <= (uint64_t)ctx->n_cu ? 8u : 4u;
  const uint32_t self = self_ok && n_cols == 1 ? 1 : 0;
  const uint32_t seq_max = std::max(base_pos + n_cols - self, 1u);   // streamed rows (position 0 alone: one empty split)
  const uint32_t tiles = ceil_div(seq_max, 32);
  const uint32_t occ = nb == 1 ? 2 : 1;
  const uint32_t target = ctx->decode_splits_override ? ctx->decode_splits_override
                                                      : std::max(1u, (occ * (uint32_t)ctx->n_cu) / (c.n_kv_heads * groups));
  uint32_t sl, ns;
  if (one_split || ctx->decode_splits_override) {
    // a given number of splits (a tuning override; its splits are contiguous ranges, the last one open-ended), or one
    const uint32_t tpw = one_split ? std::max(ceil_div(tiles, W), 1u) : std::max(ceil_div(tiles, target * W), 1u);
    sl = 32 * W * tpw; ns = ceil_div(seq_max, sl);
  } else if ((nb == 1 || (nb == 2 && W == 4 && seq_max > 32 * W)) &&
             ceil_div(seq_max, 32 * W) <= (nb == 2 && c.head_dim == 128 ? 2 * target : target)) {
    // One 16-row block and no more one-tile-per-wave splits than two workgroups a CU hold at once: the single-round
    // kernel, the whole context in flight in one go.  A single split more would run as a second round behind the
    // first (measured, MoE shape: 32768 rows 16.3 us, 32800 rows 19.7 us, against 18.8 us on the tile loop below).
    sl = 32 * W; ns = ceil_div(seq_max, sl);
  } else {
    // The tile loop, and there ONE workgroup a CU is the target whatever the row blocks: a workgroup keeps 128 KB of
    // K/V loads in flight, which saturates the memory system from half the CUs on; a second one on the CU only adds
    // its fixed costs (start-up, the merge of its waves, its partials, a longer merge pass) and, measured on read-only
    // stand-ins of the loop, lowers the stream's rate (256 MiB: 46 us with one workgroup a CU, 56 - 60 us with two).
    // Measured, one column: MoE shape at 40000 / 65536 / 131072 rows 24.2 -> 21.0, 32.6 -> 28.9, 56.3 -> 49.7 us; 27B
    // shape at 65536 rows 57.2 -> 52.6 us.  The loop deals a kv head's tiles round robin to the waves of all its
    // splits (AttnParams::tile_ilv), so any number of splits is balanced to within a tile and split_len is nominal:
    // the rows of a split's tiles, rounded up.  No floor on the tiles per wave: short and mid-length verify blocks are
    // bound by the chain of a wave's tiles, not by the bytes of the partials (a former floor of 4 / 6 / 8 tiles a wave
    // with 2 / 3 / 4 row blocks, meant to keep the partials a few percent of the K/V bytes, left most CUs without a
    // workgroup: MoE shape, 4 columns at 4096 / 8192 / 16384 rows 20.5 -> 15.9, 20.7 -> 16.3, 21.1 -> 17.7 us; dense
    // hd-128 shape, 32 columns at 4096 / 8192 rows 26.6 -> 19.0, 26.6 -> 20.4 us).
    const uint32_t target1 = std::max(1u, (uint32_t)ctx->n_cu / (c.n_kv_heads * groups));
    ns = std::max(1u, std::min(target1, tiles / W));
    // ... and the fewest splits with that many tiles per wave: 2049 tiles over 256 waves are nine rounds for one wave
    // and eight for the rest, the ninth a round trip for 16 KB; over 228 waves they are nine full rounds of fewer bytes
    // (27B shape, 8 columns at 65536: 59.6 -> 58.5 us; MoE shape, one column at 34000 / 50000 / 100000 rows: 21.3 ->
    // 19.1, 26.9 -> 24.2, 42.5 -> 40.4 us).
    const uint32_t tpw = ceil_div(tiles, ns * W);
    ns = ceil_div(tiles, tpw * W);
    sl = 32 * W * tpw;
  }
  pl->kernel = 0; pl->split_len = sl; pl->n_splits = ns;
  pl->col_groups = groups; pl->cols_per_group = cw; pl->waves = W; pl->row_blocks = nb; pl->slots = pl->n_splits + self;
  return PA_OK;
}

// Prefill (MFMA kernel): a workgroup is 8 wavefronts x 32 query rows = 256 rows of one kv head, i.e.
// floor(256 / G) columns x G heads.  Chunks wide enough to give every CU a workgroup run unsplit and write the
// output directly; narrower chunks are also split over the context (partials + merge kernel) until every CU has a
// workgroup (one is resident per CU; a second round of a few workgroups costs more than longer splits).  Chunks of fewer rows than one wavefront tile go to the split-K decode kernel.
static int plan_prefill(const pa_ctx* ctx, uint32_t base_pos, uint32_t n_cols, pa_plan* pl) {
  const pa_config& c = ctx->cfg;
  const uint32_t G = c.n_heads / c.n_kv_heads;
  const uint32_t max_rows_sk = c.head_dim == 256 ? 32u : 64u;
  if (n_cols * G <= max_rows_sk) return plan_decode(ctx, base_pos, n_cols, pl, true);
  // pa_set_prefill_tile: 2 = never the matrix-core kernel (where the split-K kernel can hold a column's heads),
  // 1 = always (the two table rules below are skipped), 0 = the table
  if (ctx->prefill_tile_mode == 2 && max_rows_sk >= G) return plan_decode(ctx, base_pos, n_cols, pl, true);
  const bool table = ctx->prefill_tile_mode == 0;
  // A chunk of a few column groups over a long context (the reference's own prefill passes are 16 columns wide) is
  // bound by the K/V stream, not by the matrix cores: the split-K kernel serves it in column groups, whose workgroups
  // share the stream through L2, for as long as groups x K/V bytes stays below what the MFMA kernel's fixed costs
  // (Q staging, one partial per split and row, the merge) amount to.  Measured crossover on the MoE and 27B shapes
  // at 32K - 64K rows: about 1.4 GB of L2-level K/V traffic; below 4096 rows both kernels take 25 - 40 us.
  if (table && n_cols * G <= 512 && base_pos + n_cols >= 4096 && max_rows_sk >= G) {
    pa_plan sk;
    const uint64_t kv_bytes = 2ull * (base_pos + n_cols) * c.n_kv_heads * c.head_dim * (kv_q8(ctx) ? 1 : 2);
    if (plan_decode(ctx, base_pos, n_cols, &sk, true) == PA_OK && (uint64_t)sk.col_groups * kv_bytes <= 1400000000ull) {
      *pl = sk;
      return PA_OK;
    }
  }
  // A small chunk (the first chunks of a prompt, a 512-column chunk over a 2K context): the matrix-core kernel's
  // 256-row workgroups leave most CUs idle unless the chunk is also split over the context, and then the partials
  // (a row of head_dim floats per split and stacked row) and the merge launch cost more than the attention itself.
  // Below about 8 GFLOP of causal work the split-K kernel serves the chunk in one launch instead: 16- or 32-row
  // workgroups (the larger that still gives every CU a workgroup), each over the whole context of its columns,
  // writing the normalised, gated output itself -- for contexts below 4096 rows (longer ones are the rule above) and
  // chunks whose column groups fill at least half the chip.  Measured crossover (us per call, this path vs the matrix-core
  // kernel): dense shape 256 columns from position 0: 6.3 vs 16.8, 512 columns at 1536: 25 vs 32, 2048 from 0: 48 vs
  // 47; MoE shape 256 from 0: 11 vs 33, 512 from 0: 21 vs 36, 1024 from 0: 52 vs 44.
  {
    const double flops = 4.0 * c.n_heads * c.head_dim * ((double)n_cols * base_pos + 0.5 * (double)n_cols * (n_cols + 1));
    if (table && flops <= 8.0e9 && G <= 16 && base_pos + n_cols < 4096 && !ctx->decode_splits_override) {
      const uint32_t rows = (uint64_t)ceil_div(n_cols, 32 / G) * c.n_kv_heads >= (uint64_t)ctx->n_cu ? 32u : 16u;
      // one split per workgroup only pays when the column groups alone occupy the chip (or the context is a few tiles)
      if ((uint64_t)ceil_div(n_cols, rows / G) * c.n_kv_heads * 2 >= (uint64_t)ctx->n_cu || base_pos + n_cols <= 256)
        return plan_decode(ctx, base_pos, n_cols, pl, true, rows, true);
    }
  }
  const uint32_t rows_wg = 256;
  const uint32_t cw = rows_wg / G;
  if (cw == 0) return PA_ERR_UNSUPPORTED;
  const uint32_t groups = ceil_div(n_cols, cw);
  const uint32_t seq_max = base_pos + n_cols;
  const uint32_t base_wgs = groups * c.n_kv_heads;
  uint32_t splits = 1;
  if (base_wgs < (uint32_t)ctx->n_cu) splits = std::min(std::max(1u, (uint32_t)ctx->n_cu / base_wgs), std::max(1u, seq_max / 256));
  uint32_t sl = ceil_div(ceil_div(seq_max, splits), 32) * 32;
  pl->kernel = 1; pl->split_len = sl; pl->n_splits = ceil_div(seq_max, sl);
  pl->col_groups = groups; pl->cols_per_group = cw; pl->waves = 8; pl->row_blocks = 8; pl->slots = pl->n_splits;
  return PA_OK;
}

extern "C" int pa_plan_query(const pa_ctx* ctx, int kind, uint32_t base_pos, uint32_t n_cols, pa_plan* out) {
  if (!ctx || !out || n_cols == 0) return PA_ERR_INVALID;
  return kind == 0 ? plan_decode(ctx, base_pos, n_cols, out) : plan_prefill(ctx, base_pos, n_cols, out);
}
extern "C" int pa_set_prefill_tile(pa_ctx* ctx, int mode) {
  if (!ctx) return PA_ERR_INVALID;
  if (mode < 0 || mode > 2) return fail(ctx, PA_ERR_INVALID, "pa_set_prefill_tile: mode must be 0 (table), 1 (always) or 2 (never)");
  ctx->prefill_tile_mode = mode;
  return PA_OK;
}
extern "C" int pa_set_decode_splits(pa_ctx* ctx, uint32_t splits) {
  if (!ctx) return PA_ERR_INVALID;
  ctx->decode_splits_override = splits;
  return PA_OK;
}

// ---- attention ----------------------------------------------------------------------------------

// Context scratch (split partials, projection and chunk buffers, the int8 staging cache) grows on demand and is never
// freed or moved while the context lives: launches recorded into a HIP graph by the caller carry the address they
// were recorded with, and a later, larger pass must not pull that memory from under a replay.  The outgrown block is
// kept until pa_destroy.  (Growth itself allocates, so a pass that grows a buffer cannot be captured; one eager call
// of the same or a larger shape before the capture is enough.)
static int grow_scratch(pa_ctx* ctx, void** buf, size_t* have, size_t need) {
  if (need <= *have) return PA_OK;
  void* mem = nullptr;
  HIPCHK(ctx, hipMalloc(&mem, need));
  if (*buf) ctx->retired.push_back(*buf);
  *buf = mem; *have = need;
  return PA_OK;
}

static int ensure_partials(pa_ctx* ctx, uint32_t n_cols, uint32_t slots) {
  const pa_config& c = ctx->cfg;
  const size_t need_o = (size_t)n_cols * c.n_heads * slots * c.head_dim * sizeof(float);
  const size_t need_ml = (size_t)n_cols * c.n_heads * slots * 2 * sizeof(float);
  int rc = grow_scratch(ctx, (void**)&ctx->part_o, &ctx->part_o_bytes, need_o);
  if (rc) return rc;
  return grow_scratch(ctx, (void**)&ctx->part_ml, &ctx->part_ml_bytes, need_ml);
}

// an event pair for a kernel-exact timing of the next main-kernel launch (profiling on), else an empty PaTiming
static int prof_pair(pa_ctx* ctx, PaTiming* t) {
  *t = PaTiming();
  if (!ctx->profiling) return PA_OK;
  if (ctx->prof_used + 2 > ctx->prof_events.size()) {
    for (int i = 0; i < 2; i++) { hipEvent_t ev; HIPCHK(ctx, hipEventCreate(&ev)); ctx->prof_events.push_back(ev); }
  }
  t->start = ctx->prof_events[ctx->prof_used]; t->stop = ctx->prof_events[ctx->prof_used + 1];
  ctx->prof_used += 2;
  return PA_OK;
}

// While profiling, the merge launch of a call is stamped as well (a pair of its own that nobody reads; one pair per
// profiled call, reset with the main pairs): a dispatch that carries stamps is handled differently from one that does
// not, and with only the main kernel stamped its own stamps read 0.7 - 1.5 us more than a kernel trace -- where every
// dispatch carries them -- reports.
static int prof_aux_pair(pa_ctx* ctx, const PaTiming& main, PaTiming* t) {
  *t = PaTiming();
  if (!main.start) return PA_OK;
  if (ctx->prof_aux_used + 2 > ctx->prof_aux.size()) {
    for (int i = 0; i < 2; i++) { hipEvent_t ev; HIPCHK(ctx, hipEventCreate(&ev)); ctx->prof_aux.push_back(ev); }
  }
  t->start = ctx->prof_aux[ctx->prof_aux_used]; t->stop = ctx->prof_aux[ctx->prof_aux_used + 1];
  ctx->prof_aux_used += 2;
  return PA_OK;
}

static int attn_common(pa_ctx* ctx, const char* who, int kind, uint32_t layer, const float* d_q, uint32_t q_stride,
                       const float* d_gate, uint32_t gate_stride, uint32_t base_pos, uint32_t n_cols, void* d_out,
                       uint32_t out_stride, int out_dtype) {
  if (!ctx) return PA_ERR_INVALID;
  int rc = check_cols(ctx, who, layer, true, base_pos, n_cols);
  if (rc) return rc;
  const pa_config& c = ctx->cfg;
  const uint32_t qd = c.n_heads * c.head_dim;
  if (!d_out) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null output");
  if (out_dtype != PA_OUT_F32 && out_dtype != PA_OUT_F16) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": bad out_dtype");
  if (!d_q) { d_q = ctx->q_buf; q_stride = qd; }
  if (q_stride < qd || out_stride < qd || (d_gate && gate_stride < qd))
    return fail(ctx, PA_ERR_INVALID, std::string(who) + ": column stride shorter than a column");
  if ((q_stride & 3) || (out_stride & 3) || (d_gate && (gate_stride & 3)) || ((uintptr_t)d_q & 15) || ((uintptr_t)d_out & 15) || ((uintptr_t)d_gate & 15))
    return fail(ctx, PA_ERR_INVALID, std::string(who) + ": buffers must be 16-byte aligned with strides a multiple of 4 elements");
  if (kind == 0 && n_cols > 1 && (c.flags & PA_FLAG_VERIFY_EXACT)) {
    // column-exact verify: every column is the one-column decode at its own position (its own splits, its own row
    // block), so its bits are those of a sequential decode.
    // A run of columns with the same one-column plan is ONE pass: every column a column group of its own, each
    // workgroup doing exactly what the one-column launch at that column's position does -- same splits, same row
    // order, own row as a partial -- and the wavefront merge over the columns.  The columns' workgroups of a (split,
    // kv head) run side by side on one XCD and share the rows in its L2, so the cache is read from HBM about once.
    // The plan moves at few positions (a split more on the single-round kernel every 128 rows, a tile per wave more
    // on the tile loop every few thousand), so a block is one run, or two.
    auto one_col_plan = [&](uint32_t pos, pa_plan* pl) -> bool {
      return plan_decode(ctx, pos, 1, pl, true) == PA_OK && pl->kernel == 0 && pl->row_blocks == 1 && pl->waves == 4 && plan_self_row(*pl) &&
             pl->slots <= 8192;
    };
    // (round-robin tiles: the split length is nominal, the splits are the same whenever their number is)
    auto same_plan = [&](const pa_plan& a, const pa_plan& b) -> bool {
      return (a.split_len == b.split_len || (plan_tile_ilv(a) && plan_tile_ilv(b))) && a.n_splits == b.n_splits && a.slots == b.slots;
    };
    const size_t osz = out_dtype == PA_OUT_F16 ? 2 : 4;
    for (uint32_t col = 0; col < n_cols;) {
      pa_plan p0, p1;
      uint32_t run = 1;
      if (one_col_plan(base_pos + col, &p0))
        while (col + run < n_cols && run < 65535 && one_col_plan(base_pos + col + run, &p1) && same_plan(p0, p1)) run++;
      const float* q_c = d_q + (size_t)col * q_stride;
      const float* gate_c = d_gate ? d_gate + (size_t)col * gate_stride : nullptr;
      void* out_c = (unsigned char*)d_out + (size_t)col * out_stride * osz;
      if (run == 1) {                 // a column on its own: the one-column decode itself
        if ((rc = attn_common(ctx, who, 0, layer, q_c, q_stride, gate_c, gate_stride, base_pos + col, 1, out_c, out_stride, out_dtype))) return rc;
      } else {
        if ((rc = ensure_partials(ctx, run, p0.slots))) return rc;
        AttnParams p; memset(&p, 0, sizeof p);
        p.q = q_c; p.gate = gate_c; p.k_cache = ctx->layers[layer].k; p.v_cache = ctx->layers[layer].v;
        p.k_scale = ctx->layers[layer].ks; p.v_scale = ctx->layers[layer].vs;
        p.part_o = ctx->part_o; p.part_ml = ctx->part_ml; p.out = out_c;
        p.q_stride = q_stride; p.gate_stride = gate_stride; p.out_stride = out_stride;
        p.n_heads = c.n_heads; p.n_kv_heads = c.n_kv_heads; p.group = c.n_heads / c.n_kv_heads;
        p.base_pos = base_pos + col; p.n_cols = run;
        p.split_len = p0.split_len; p.n_splits = p0.n_splits; p.slots = p0.slots; p.cols_per_group = 1;
        p.self_row = 1; p.part_f16 = plan_f16_partials(p0, 1); p.exact_cols = 1; p.tile_ilv = plan_tile_ilv(p0);
        p.max_seq = c.max_seq; p.out_f16 = out_dtype == PA_OUT_F16;
        p.scale = (float)(1.0 / std::sqrt((double)c.head_dim));
        p.gate_head_stride = c.head_dim;
        PaTiming tm, tm2;
        if ((rc = prof_pair(ctx, &tm))) return rc;
        HIPCHK(ctx, pa_launch_decode(p, c.head_dim, 1, 4, run, ctx->stream, &tm));
        if ((rc = prof_aux_pair(ctx, tm, &tm2))) return rc;
        HIPCHK(ctx, pa_launch_combine(p, c.head_dim, ctx->stream, &tm2));
      }
      col += run;
    }
    return PA_OK;
  }
  pa_plan pl;
  rc = kind == 0 ? plan_decode(ctx, base_pos, n_cols, &pl, true) : plan_prefill(ctx, base_pos, n_cols, &pl);
  if (rc) return fail(ctx, rc, std::string(who) + ": shape outside the gfx950 table");
  if (pl.slots > 8192) return fail(ctx, PA_ERR_UNSUPPORTED, std::string(who) + ": too many splits");
  // one split and no own-row partial: the kernel writes the output itself (the prefill kernel, or the split-K kernel's
  // tile loop: its single-round form always leaves a partial)
  const bool direct = pl.n_splits == 1 && !plan_self_row(pl) && (pl.kernel == 1 || pl.split_len != 32 * pl.waves || pl.row_blocks > 1);
  if (!direct && (rc = ensure_partials(ctx, n_cols, pl.slots))) return rc;
  AttnParams p; memset(&p, 0, sizeof p);
  p.q = d_q; p.gate = d_gate; p.k_cache = ctx->layers[layer].k; p.v_cache = ctx->layers[layer].v;
  p.part_o = ctx->part_o; p.part_ml = ctx->part_ml; p.out = d_out;
  p.q_stride = q_stride; p.gate_stride = gate_stride; p.out_stride = out_stride;
  p.n_heads = c.n_heads; p.n_kv_heads = c.n_kv_heads; p.group = c.n_heads / c.n_kv_heads;
  p.base_pos = base_pos; p.n_cols = n_cols;
  p.k_scale = ctx->layers[layer].ks; p.v_scale = ctx->layers[layer].vs;
  if (pl.kernel == 1 && kv_q8(ctx)) {
    // int8 caches under the MFMA prefill kernel (the reference has no tiled prefill for them): the rows the chunk can
    // see are widened once into a context-owned f16 staging cache of one layer's size -- a few percent of the
    // chunk's attention time -- and the f16 kernel runs on that.  Rows past the chunk's last position up to the
    // next multiple of 32 are staged as zeros.
    const size_t wide_elems = ((size_t)c.max_seq + 32) * c.n_kv_heads * c.head_dim;
    for (uint16_t** w : {&ctx->wide_k, &ctx->wide_v}) {
      if (*w) continue;
      uint16_t* mem = nullptr;                       // the padding rows from max_seq on stay zero for good
      HIPCHK(ctx, hipMalloc((void**)&mem, wide_elems * sizeof(uint16_t)));
      hipError_t e = hipMemsetAsync(mem, 0, wide_elems * sizeof(uint16_t), ctx->stream);
      if (e != hipSuccess) { (void)hipFree(mem); HIPCHK(ctx, e); }
      *w = mem;
    }
    const uint32_t live = base_pos + n_cols, staged = std::min(ceil_div(live, 32) * 32, c.max_seq + 32);
    HIPCHK(ctx, pa_launch_widen_q8(ctx->layers[layer].k, ctx->layers[layer].v, ctx->layers[layer].ks, ctx->layers[layer].vs, ctx->wide_k,
                                   ctx->wide_v, c.n_kv_heads, c.head_dim, c.max_seq + 32, live, staged, ctx->stream));
    p.k_cache = ctx->wide_k; p.v_cache = ctx->wide_v; p.k_scale = nullptr; p.v_scale = nullptr;
  }
  p.split_len = pl.split_len; p.n_splits = pl.n_splits; p.slots = pl.slots; p.cols_per_group = pl.cols_per_group;
  p.self_row = plan_self_row(pl) ? 1 : 0;
  p.direct_out = direct && pl.kernel == 0 ? 1 : 0;
  p.part_f16 = !direct && plan_f16_partials(pl, n_cols);
  p.tile_ilv = plan_tile_ilv(pl);
  p.single_round2 = plan_single_round2(pl);
  p.max_seq = c.max_seq; p.out_f16 = out_dtype == PA_OUT_F16;
  p.scale = (float)(1.0 / std::sqrt((double)c.head_dim));
  p.gate_head_stride = c.head_dim;
  PaTiming tm;
  if ((rc = prof_pair(ctx, &tm))) return rc;
  if (pl.kernel == 0) HIPCHK(ctx, pa_launch_decode(p, c.head_dim, pl.row_blocks, pl.waves, pl.col_groups, ctx->stream, &tm));
  else HIPCHK(ctx, pa_launch_prefill(p, c.head_dim, pl.row_blocks, pl.col_groups, ctx->stream, &tm));
  if (!direct) {
    PaTiming tm2;
    if ((rc = prof_aux_pair(ctx, tm, &tm2))) return rc;
    HIPCHK(ctx, pa_launch_combine(p, c.head_dim, ctx->stream, &tm2));
  }
  return PA_OK;
}

extern "C" int pa_attn_decode(pa_ctx* ctx, uint32_t layer, const float* d_q, uint32_t q_stride, const float* d_gate,
                              uint32_t gate_stride, uint32_t base_pos, uint32_t n_cols, void* d_out, uint32_t out_stride,
                              int out_dtype) {
  return attn_common(ctx, "pa_attn_decode", 0, layer, d_q, q_stride, d_gate, gate_stride, base_pos, n_cols, d_out, out_stride, out_dtype);
}
extern "C" int pa_attn_prefill(pa_ctx* ctx, uint32_t layer, const float* d_q, uint32_t q_stride, const float* d_gate,
                               uint32_t gate_stride, uint32_t base_pos, uint32_t n_cols, void* d_out, uint32_t out_stride,
                               int out_dtype) {
  return attn_common(ctx, "pa_attn_prefill", 1, layer, d_q, q_stride, d_gate, gate_stride, base_pos, n_cols, d_out, out_stride, out_dtype);
}

// static_scratch: the partials go to the library's file-scope device array and the call allocates nothing
static int decode_step_common(pa_ctx* ctx, const char* who, bool static_scratch, uint32_t layer, const float* d_q_in, const float* d_k,
                              const float* d_v, const float* d_qw, const float* d_kw, uint32_t pos, void* d_out, int out_dtype) {
  if (!ctx) return PA_ERR_INVALID;
  int rc = check_cols(ctx, who, layer, true, pos, 1);
  if (rc) return rc;
  const pa_config& c = ctx->cfg;
  const bool gated = (c.flags & PA_FLAG_GATE) != 0, norm = (c.flags & PA_FLAG_QK_NORM) != 0;
  if (!d_q_in || !d_k || !d_v || !d_out) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null buffer");
  if (norm && (!d_qw || !d_kw)) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": norm weights required");
  if (out_dtype != PA_OUT_F32 && out_dtype != PA_OUT_F16) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": bad out_dtype");
  if (((uintptr_t)d_q_in & 15) || ((uintptr_t)d_k & 15) || ((uintptr_t)d_v & 15) || ((uintptr_t)d_out & 15))
    return fail(ctx, PA_ERR_INVALID, std::string(who) + ": buffers must be 16-byte aligned");
  if (c.n_heads / c.n_kv_heads > 16) return fail(ctx, PA_ERR_UNSUPPORTED, std::string(who) + ": more than 16 query heads per kv head");
  pa_plan pl;
  rc = plan_decode(ctx, pos, 1, &pl, true);
  if (rc) return fail(ctx, rc, std::string(who) + ": shape outside the gfx950 table");
  if (pl.slots > 8192) return fail(ctx, PA_ERR_UNSUPPORTED, std::string(who) + ": too many splits");
  if (pl.row_blocks != 1 || pl.waves != 4 || pl.col_groups != 1 || !plan_self_row(pl)) return fail(ctx, PA_ERR_UNSUPPORTED, std::string(who) + ": plan is not a one-block decode");
  float* part_o = nullptr; float* part_ml = nullptr;
  if (static_scratch) {
    const size_t need_o = ((size_t)c.n_heads * pl.slots * c.head_dim * sizeof(float) + 255) & ~(size_t)255;
    const size_t need_ml = (size_t)c.n_heads * pl.slots * 2 * sizeof(float);
    if (need_o + need_ml > PA_STATIC_SCRATCH_BYTES)
      return fail(ctx, PA_ERR_UNSUPPORTED, std::string(who) + ": the split partials of this shape (" + std::to_string(need_o + need_ml) +
                  " bytes) exceed the library's static scratch (" + std::to_string(PA_STATIC_SCRATCH_BYTES) + " bytes); use pa_attn_decode_step");
    part_o = (float*)ctx->static_scratch; part_ml = (float*)((unsigned char*)ctx->static_scratch + need_o);
  } else {
    if ((rc = ensure_partials(ctx, 1, pl.slots))) return rc;
    part_o = ctx->part_o; part_ml = ctx->part_ml;
  }
  AttnParams p; memset(&p, 0, sizeof p);
  p.k_cache = ctx->layers[layer].k; p.v_cache = ctx->layers[layer].v;
  p.k_scale = ctx->layers[layer].ks; p.v_scale = ctx->layers[layer].vs;
  p.part_o = part_o; p.part_ml = part_ml; p.out = d_out;
  p.n_heads = c.n_heads; p.n_kv_heads = c.n_kv_heads; p.group = c.n_heads / c.n_kv_heads;
  p.base_pos = pos; p.n_cols = 1;
  p.split_len = pl.split_len; p.n_splits = pl.n_splits; p.slots = pl.slots; p.cols_per_group = pl.cols_per_group;
  p.self_row = 1; p.part_f16 = plan_f16_partials(pl, 1); p.tile_ilv = plan_tile_ilv(pl);
  p.max_seq = c.max_seq; p.out_f16 = out_dtype == PA_OUT_F16;
  p.scale = (float)(1.0 / std::sqrt((double)c.head_dim));
  // the pre-step inputs; the gate is read in place from the interleaved [q | gate] heads
  p.f_q_in = d_q_in; p.f_k_in = d_k; p.f_v_in = d_v;
  p.f_qw = norm ? d_qw : nullptr; p.f_kw = norm ? d_kw : nullptr;
  p.rope_tab = ctx->rope_tab; p.inv_freq = ctx->inv_freq;
  p.f_q_head_stride = c.head_dim * (gated ? 2 : 1); p.n_rot = c.n_rot; p.eps = c.eps;
  p.gate = gated ? d_q_in + c.head_dim : nullptr;
  p.gate_head_stride = p.f_q_head_stride;
  PaTiming tm;                                        // profiling may create events: not on the allocation-free path
  if (!static_scratch && (rc = prof_pair(ctx, &tm))) return rc;
  HIPCHK(ctx, pa_launch_decode_step(p, c.head_dim, ctx->stream, &tm));
  PaTiming tm2;
  if ((rc = prof_aux_pair(ctx, tm, &tm2))) return rc;
  HIPCHK(ctx, pa_launch_combine(p, c.head_dim, ctx->stream, &tm2));
  return PA_OK;
}

extern "C" int pa_attn_decode_step(pa_ctx* ctx, uint32_t layer, const float* d_q_in, const float* d_k, const float* d_v,
                                   const float* d_qw, const float* d_kw, uint32_t pos, void* d_out, int out_dtype) {
  return decode_step_common(ctx, "pa_attn_decode_step", false, layer, d_q_in, d_k, d_v, d_qw, d_kw, pos, d_out, out_dtype);
}
extern "C" int pa_attn_decode_step_noalloc(pa_ctx* ctx, uint32_t layer, const float* d_q_in, const float* d_k, const float* d_v,
                                           const float* d_qw, const float* d_kw, uint32_t pos, void* d_out, int out_dtype) {
  return decode_step_common(ctx, "pa_attn_decode_step_noalloc", true, layer, d_q_in, d_k, d_v, d_qw, d_kw, pos, d_out, out_dtype);
}

// ---- projections (one-token passes) -------------------------------------------------------------

extern "C" int pa_weight_create(pa_ctx* ctx, int kind, uint32_t d_out, uint32_t d_in, const void* h_w, const void* h_scales, pa_weight** out) {
  const char* who = "pa_weight_create";
  if (!ctx || !out) return PA_ERR_INVALID;
  *out = nullptr;
  if (kind != PA_W_F32 && kind != PA_W_Q8_0 && kind != PA_W_Q4_0) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": unknown weight kind");
  if (!h_w || (kind != PA_W_F32 && !h_scales)) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null plane");
  if (d_out == 0 || d_in == 0 || (d_in & 31)) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": d_in must be a positive multiple of 32");
  if (d_in > 8192u) return fail(ctx, PA_ERR_UNSUPPORTED, std::string(who) + ": d_in beyond the gfx950 table");
  pa_weight* w = new (std::nothrow) pa_weight();
  if (!w) return fail(ctx, PA_ERR_NOMEM, std::string(who) + ": out of host memory");
  w->kind = kind; w->d_out = d_out; w->d_in = d_in;
  const size_t wbytes = kind == PA_W_F32 ? (size_t)d_out * d_in * 4 : kind == PA_W_Q8_0 ? (size_t)d_out * d_in : (size_t)d_out * d_in / 2;
  const size_t sbytes = kind == PA_W_F32 ? 0 : (size_t)d_out * (d_in / 32) * 2;
  hipError_t e = hipMalloc(&w->w, wbytes);
  if (e == hipSuccess && sbytes) e = hipMalloc((void**)&w->scales, sbytes);
  if (e == hipSuccess) e = hipMemcpyAsync(w->w, h_w, wbytes, hipMemcpyHostToDevice, ctx->stream);
  if (e == hipSuccess && sbytes) e = hipMemcpyAsync(w->scales, h_scales, sbytes, hipMemcpyHostToDevice, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  if (e != hipSuccess) {
    if (w->w) (void)hipFree(w->w);
    if (w->scales) (void)hipFree(w->scales);
    delete w;
    return fail_hip(ctx, e, "pa_weight_create: upload");
  }
  *out = w;
  return PA_OK;
}

extern "C" int pa_weight_destroy(pa_ctx* ctx, pa_weight* w) {
  if (!ctx) return PA_ERR_INVALID;
  if (!w) return PA_OK;
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  if (w->w) (void)hipFree(w->w);
  if (w->scales) (void)hipFree(w->scales);
  if (w->w16_ready) (void)hipEventDestroy(w->w16_ready);
  if (w->w16) { (void)hipFree(w->w16); ctx->weight_cache_used -= std::min(ctx->weight_cache_used, w->w16_bytes); }
  delete w;
  return PA_OK;
}

extern "C" int pa_set_weight_cache(pa_ctx* ctx, size_t max_bytes) {
  if (!ctx) return PA_ERR_INVALID;
  ctx->weight_cache_limit = max_bytes;
  return PA_OK;
}

static int gemv_common(pa_ctx* ctx, const char* who, const pa_weight* w, const float* d_x, const float* d_norm_w, float* d_xn_out, float* d_y, int acc) {
  if (!ctx) return PA_ERR_INVALID;
  if (!w || !d_x || !d_y) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null argument");
  if (((uintptr_t)d_x & 15) || ((uintptr_t)d_norm_w & 15) || ((uintptr_t)d_xn_out & 15))
    return fail(ctx, PA_ERR_INVALID, std::string(who) + ": vectors must be 16-byte aligned");
  GemvParams p; memset(&p, 0, sizeof p);
  p.w = w->w; p.scales = w->scales; p.x = d_x; p.norm_w = d_norm_w; p.xn_out = d_xn_out; p.y = d_y;
  p.d_out = w->d_out; p.d_in = w->d_in; p.eps = ctx->cfg.eps; p.acc = acc; p.kind = w->kind;
  HIPCHK(ctx, pa_launch_gemv(p, ctx->n_cu, ctx->stream));
  return PA_OK;
}

extern "C" int pa_gemv(pa_ctx* ctx, const pa_weight* w, const float* d_x, float* d_y, int acc) {
  return gemv_common(ctx, "pa_gemv", w, d_x, nullptr, nullptr, d_y, acc);
}
extern "C" int pa_gemv_norm(pa_ctx* ctx, const pa_weight* w, const float* d_x_raw, const float* d_norm_w, float* d_xn_out, float* d_y) {
  if (ctx && !d_norm_w) return fail(ctx, PA_ERR_INVALID, "pa_gemv_norm: null norm weight");
  return gemv_common(ctx, "pa_gemv_norm", w, d_x_raw, d_norm_w, d_xn_out, d_y, 0);
}

extern "C" int pa_attn_layer_decode(pa_ctx* ctx, uint32_t layer, const pa_weight* w_qkv, const pa_weight* w_o, const float* d_attn_norm_w,
                                    const float* d_qw, const float* d_kw, float* d_x, uint32_t pos) {
  const char* who = "pa_attn_layer_decode";
  if (!ctx) return PA_ERR_INVALID;
  const pa_config& c = ctx->cfg;
  if (!w_qkv || !w_o || !d_attn_norm_w || !d_x) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null argument");
  const uint32_t qd = c.n_heads * c.head_dim, kvd = c.n_kv_heads * c.head_dim;
  const uint32_t q_rows = qd * ((c.flags & PA_FLAG_GATE) ? 2 : 1);
  if (w_qkv->d_out != q_rows + 2 * kvd) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": w_qkv must have q (+ gate), k and v rows");
  if (w_o->d_in != qd || w_o->d_out != w_qkv->d_in) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": w_o must map n_heads x head_dim back to the model width");
  const size_t need = ((size_t)w_qkv->d_out + qd) * sizeof(float);
  int rc = grow_scratch(ctx, (void**)&ctx->proj_buf, &ctx->proj_buf_bytes, need);
  if (rc) return rc;
  float* qkv = ctx->proj_buf;
  float* attn_out = ctx->proj_buf + w_qkv->d_out;
  if ((rc = gemv_common(ctx, who, w_qkv, d_x, d_attn_norm_w, nullptr, qkv, 0))) return rc;
  if ((rc = pa_attn_decode_step(ctx, layer, qkv, qkv + q_rows, qkv + q_rows + kvd, d_qw, d_kw, pos, attn_out, PA_OUT_F32))) return rc;
  return gemv_common(ctx, who, w_o, attn_out, nullptr, nullptr, d_x, 1);
}

extern "C" int pa_rmsnorm_f16(pa_ctx* ctx, const float* d_x, uint32_t x_stride, const float* d_norm_w, uint32_t dim, uint32_t n_cols,
                              void* d_xn_f16, uint32_t xn_stride) {
  const char* who = "pa_rmsnorm_f16";
  if (!ctx) return PA_ERR_INVALID;
  if (!d_x || !d_norm_w || !d_xn_f16) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null argument");
  if (dim == 0 || (dim & 3) || n_cols == 0 || x_stride < dim || xn_stride < dim || (x_stride & 3) || (xn_stride & 3))
    return fail(ctx, PA_ERR_INVALID, std::string(who) + ": dim and strides must be positive multiples of 4, strides >= dim");
  if (((uintptr_t)d_x & 15) || ((uintptr_t)d_norm_w & 15) || ((uintptr_t)d_xn_f16 & 7))
    return fail(ctx, PA_ERR_INVALID, std::string(who) + ": buffers must be 16-byte aligned");
  HIPCHK(ctx, pa_launch_rmsnorm_f16(d_x, x_stride, d_norm_w, dim, ctx->cfg.eps, n_cols, (uint16_t*)d_xn_f16, xn_stride, ctx->stream));
  return PA_OK;
}

extern "C" int pa_gemm(pa_ctx* ctx, const pa_weight* w, const void* d_x_f16, uint32_t x_stride, uint32_t n_cols, float* d_y, uint32_t y_stride, int acc) {
  const char* who = "pa_gemm";
  if (!ctx) return PA_ERR_INVALID;
  if (!w || !d_x_f16 || !d_y) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null argument");
  if (n_cols == 0 || x_stride < w->d_in || (x_stride & 7) || y_stride < w->d_out || ((uintptr_t)d_x_f16 & 15) || ((uintptr_t)d_y & 3))
    return fail(ctx, PA_ERR_INVALID, std::string(who) + ": x stride must be a multiple of 8 halves and >= d_in, y stride >= d_out, x 16-byte aligned");
  GemmParams p; memset(&p, 0, sizeof p);
  p.w = w->w; p.scales = w->scales; p.x = (const uint16_t*)d_x_f16; p.y = d_y; p.x_stride = x_stride; p.y_stride = y_stride;
  p.d_out = w->d_out; p.d_in = w->d_in; p.n_cols = n_cols; p.acc = acc; p.kind = w->kind;
  const bool wide = pa_gemm_wide_serves(p, ctx->n_cu);
  if (wide || pa_gemm_mid_serves(p)) {
    // the weights as f16 in fragment order: a copy kept with the weight from its first large chunk on, while the
    // context's budget lasts (the handle's contents never change); past the budget, or where the allocation fails,
    // widened per call into the context's staging
    const size_t need = pa_gemm_wide_staging_bytes(w->d_out, w->d_in);
    pa_weight* wm = const_cast<pa_weight*>(w);
    void* fresh = nullptr;                        // a copy to keep, allocated by this call; attached only once its fill is queued
    if (!wm->w16 && ctx->weight_cache_used + need <= ctx->weight_cache_limit) {
      if (hipMalloc(&fresh, need) != hipSuccess) { fresh = nullptr; (void)hipGetLastError(); }
    }
    uint16_t* w16 = wm->w16 ? wm->w16 : (uint16_t*)fresh;
    bool widen = fresh != nullptr;
    if (!w16) {
      int rc = grow_scratch(ctx, &ctx->w16_buf, &ctx->w16_buf_bytes, need);
      if (rc) return rc;
      w16 = (uint16_t*)ctx->w16_buf; widen = true;
    }
    if (wm->w16 && wm->w16_ready && wm->w16_stream != ctx->stream) {
      // the kept copy was filled on another stream: wait for that fill once, on the host; from then on any stream may read it
      HIPCHK(ctx, hipEventSynchronize(wm->w16_ready));
      (void)hipEventDestroy(wm->w16_ready);
      wm->w16_ready = nullptr; wm->w16_stream = nullptr;
    }
    hipError_t e = pa_launch_gemm_wide(p, w16, widen, !wide, ctx->n_cu, ctx->stream);
    if (fresh) {
      hipEvent_t ready = nullptr;
      if (e == hipSuccess) e = hipEventCreateWithFlags(&ready, hipEventDisableTiming);
      if (e == hipSuccess) e = hipEventRecord(ready, ctx->stream);
      if (e != hipSuccess) {
        // the fill did not go out (or cannot be tracked): the handle keeps no copy, so a later call widens again
        (void)hipStreamSynchronize(ctx->stream);
        if (ready) (void)hipEventDestroy(ready);
        (void)hipFree(fresh);
        return fail_hip(ctx, e, "pa_gemm: widening the weights");
      }
      wm->w16 = (uint16_t*)fresh; wm->w16_bytes = need; wm->w16_ready = ready; wm->w16_stream = ctx->stream;
      ctx->weight_cache_used += need;
    }
    HIPCHK(ctx, e);
    return PA_OK;
  }
  HIPCHK(ctx, pa_launch_gemm(p, ctx->n_cu, ctx->stream));
  return PA_OK;
}

extern "C" int pa_attn_layer_prefill(pa_ctx* ctx, uint32_t layer, const pa_weight* w_qkv, const pa_weight* w_o, const float* d_attn_norm_w,
                                     const float* d_qw, const float* d_kw, float* d_x, uint32_t x_stride, uint32_t base_pos, uint32_t n_cols) {
  const char* who = "pa_attn_layer_prefill";
  if (!ctx) return PA_ERR_INVALID;
  const pa_config& c = ctx->cfg;
  if (!w_qkv || !w_o || !d_attn_norm_w || !d_x) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null argument");
  int rc = check_cols(ctx, who, layer, true, base_pos, n_cols);
  if (rc) return rc;
  const uint32_t qd = c.n_heads * c.head_dim, kvd = c.n_kv_heads * c.head_dim, dim = w_qkv->d_in;
  const bool gated = (c.flags & PA_FLAG_GATE) != 0;
  const uint32_t q_rows = qd * (gated ? 2 : 1), rows = q_rows + 2 * kvd;
  if (w_qkv->d_out != rows) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": w_qkv must have q (+ gate), k and v rows");
  if (w_o->d_in != qd || w_o->d_out != dim) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": w_o must map n_heads x head_dim back to the model width");
  if (x_stride < dim || (x_stride & 3) || (dim & 7)) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": residual stride must be a multiple of 4 floats and >= the model width");
  // chunk scratch: xn f16 [cols][dim] | qkv f32 [cols][rows] | attnOut f16 [cols][qd], each 256-byte aligned
  auto up256 = [](size_t b) { return (b + 255) & ~(size_t)255; };
  const size_t b_xn = up256((size_t)n_cols * dim * 2), b_qkv = up256((size_t)n_cols * rows * 4), b_at = up256((size_t)n_cols * qd * 2);
  if ((rc = grow_scratch(ctx, &ctx->chunk_buf, &ctx->chunk_buf_bytes, b_xn + b_qkv + b_at))) return rc;
  uint16_t* xn = (uint16_t*)ctx->chunk_buf;
  float* qkv = (float*)((unsigned char*)ctx->chunk_buf + b_xn);
  uint16_t* at = (uint16_t*)((unsigned char*)ctx->chunk_buf + b_xn + b_qkv);
  if ((rc = pa_rmsnorm_f16(ctx, d_x, x_stride, d_attn_norm_w, dim, n_cols, xn, dim))) return rc;
  if ((rc = pa_gemm(ctx, w_qkv, xn, dim, n_cols, qkv, rows, 0))) return rc;
  if ((rc = pa_glue_kv(ctx, layer, qkv, rows, qkv + q_rows, rows, qkv + q_rows + kvd, rows, d_qw, d_kw, base_pos, n_cols))) return rc;
  if ((rc = pa_attn_prefill(ctx, layer, nullptr, 0, gated ? ctx->gate_buf : nullptr, qd, base_pos, n_cols, at, qd, PA_OUT_F16))) return rc;
  return pa_gemm(ctx, w_o, at, qd, n_cols, d_x, x_stride, 1);
}

// ---- cache access ---------------------------------------------------------------------------------

// The caches are head-major on the device ([nKV][max_seq + 32][hd]: every kv head's rows are one contiguous
// stream for the attention kernels); the host view of pa_kv_read / pa_kv_write stays the engine's position-major
// [rows][nKV * hd], so each call is one strided copy per kv head.
static int kv_copy(pa_ctx* ctx, const char* who, uint32_t layer, int which, uint32_t row0, uint32_t n_rows, void* host, bool to_host) {
  if (layer >= ctx->cfg.n_layers || !ctx->layers[layer].k) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": layer not allocated");
  if (which < 0 || which >= n_tensors(ctx)) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": which must be 0 (K) or 1 (V), or 2 / 3 (their scales) on an int8 cache");
  if ((uint64_t)row0 + n_rows > ctx->cfg.max_seq) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": rows exceed max_seq");
  if (!host) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null host buffer");
  if (n_rows == 0) return PA_OK;
  const pa_config& c = ctx->cfg;
  const size_t hd_bytes = head_row_bytes(ctx, which), host_pitch = hd_bytes * c.n_kv_heads, head_rows = (size_t)c.max_seq + 32;
  unsigned char* dev = (unsigned char*)ctx->layers[layer].tensor(which);
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  // one contiguous transfer per kv head through a host staging plane (a pitched copy of 512-byte rows is far slower)
  std::vector<unsigned char> plane((size_t)n_rows * hd_bytes);
  for (uint32_t g = 0; g < c.n_kv_heads; g++) {
    unsigned char* d = dev + ((size_t)g * head_rows + row0) * hd_bytes;
    unsigned char* h = (unsigned char*)host + (size_t)g * hd_bytes;
    if (to_host) {
      HIPCHK(ctx, hipMemcpy(plane.data(), d, plane.size(), hipMemcpyDeviceToHost));
      for (uint32_t r = 0; r < n_rows; r++) memcpy(h + (size_t)r * host_pitch, plane.data() + (size_t)r * hd_bytes, hd_bytes);
    } else {
      for (uint32_t r = 0; r < n_rows; r++) memcpy(plane.data() + (size_t)r * hd_bytes, h + (size_t)r * host_pitch, hd_bytes);
      HIPCHK(ctx, hipMemcpy(d, plane.data(), plane.size(), hipMemcpyHostToDevice));
    }
  }
  return PA_OK;
}
extern "C" size_t pa_kv_row_bytes(const pa_ctx* ctx, int which) {
  if (!ctx || which < 0 || which >= n_tensors(ctx)) return 0;
  return head_row_bytes(ctx, which) * ctx->cfg.n_kv_heads;
}
extern "C" int pa_kv_read(pa_ctx* ctx, uint32_t layer, int which, uint32_t row0, uint32_t n_rows, void* h_dst) {
  if (!ctx) return PA_ERR_INVALID;
  return kv_copy(ctx, "pa_kv_read", layer, which, row0, n_rows, h_dst, true);
}
extern "C" int pa_kv_write(pa_ctx* ctx, uint32_t layer, int which, uint32_t row0, uint32_t n_rows, const void* h_src) {
  if (!ctx) return PA_ERR_INVALID;
  return kv_copy(ctx, "pa_kv_write", layer, which, row0, n_rows, const_cast<void*>(h_src), false);
}
extern "C" int pa_attn_decode_gather(pa_ctx* ctx, uint32_t layer, const float* d_q, uint32_t q_stride, const float* d_gate,
                                     uint32_t gate_stride, const uint32_t* d_sel, uint32_t sel_stride, uint32_t max_rows,
                                     uint32_t n_cols, void* d_out, uint32_t out_stride, int out_dtype) {
  const char* who = "pa_attn_decode_gather";
  if (!ctx) return PA_ERR_INVALID;
  int rc = check_cols(ctx, who, layer, true, 0, n_cols);
  if (rc) return rc;
  const pa_config& c = ctx->cfg;
  const uint32_t qd = c.n_heads * c.head_dim;
  if (kv_q8(ctx)) return fail(ctx, PA_ERR_UNSUPPORTED, std::string(who) + ": no gather mode on int8 caches");
  if (!d_out || !d_sel) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null buffer");
  if (max_rows == 0 || max_rows > c.max_seq) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": max_rows must be in [1, max_seq]");
  if (sel_stride < max_rows + 1) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": sel_stride shorter than a list of max_rows");
  if (out_dtype != PA_OUT_F32 && out_dtype != PA_OUT_F16) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": bad out_dtype");
  if (!d_q) { d_q = ctx->q_buf; q_stride = qd; }
  if (q_stride < qd || out_stride < qd || (d_gate && gate_stride < qd))
    return fail(ctx, PA_ERR_INVALID, std::string(who) + ": column stride shorter than a column");
  if ((q_stride & 3) || (out_stride & 3) || (d_gate && (gate_stride & 3)) || ((uintptr_t)d_q & 15) || ((uintptr_t)d_out & 15) || ((uintptr_t)d_gate & 15) || ((uintptr_t)d_sel & 3))
    return fail(ctx, PA_ERR_INVALID, std::string(who) + ": buffers must be 16-byte aligned with strides a multiple of 4 elements");
  if (c.n_heads / c.n_kv_heads > 16) return fail(ctx, PA_ERR_UNSUPPORTED, std::string(who) + ": more than 16 query heads per kv head");
  // splits over list positions: the table's choice for one column of max_rows rows (an identity list then runs
  // exactly the dense decode), thinned when several columns share the chip
  pa_plan pl;
  rc = plan_decode(ctx, max_rows - 1, 1, &pl, false);
  if (rc) return fail(ctx, rc, std::string(who) + ": shape outside the gfx950 table");
  if (n_cols > 1 && pl.n_splits > 1) {
    const uint32_t want = std::max(1u, pl.n_splits / n_cols);
    pl.split_len = ceil_div(ceil_div(max_rows, want), 128) * 128;
    pl.n_splits = ceil_div(max_rows, pl.split_len);
  }
  pl.slots = pl.n_splits;
  if ((rc = ensure_partials(ctx, n_cols, pl.slots))) return rc;
  AttnParams p; memset(&p, 0, sizeof p);
  p.q = d_q; p.gate = d_gate; p.k_cache = ctx->layers[layer].k; p.v_cache = ctx->layers[layer].v;
  p.part_o = ctx->part_o; p.part_ml = ctx->part_ml; p.out = d_out;
  p.q_stride = q_stride; p.gate_stride = gate_stride; p.out_stride = out_stride;
  p.n_heads = c.n_heads; p.n_kv_heads = c.n_kv_heads; p.group = c.n_heads / c.n_kv_heads;
  p.base_pos = 0; p.n_cols = n_cols;
  p.split_len = pl.split_len; p.n_splits = pl.n_splits; p.slots = pl.slots; p.cols_per_group = 1;
  p.max_seq = c.max_seq; p.out_f16 = out_dtype == PA_OUT_F16;
  p.scale = (float)(1.0 / std::sqrt((double)c.head_dim));
  p.gate_head_stride = c.head_dim;
  p.sel = d_sel; p.sel_stride = sel_stride; p.sel_max = std::min(max_rows, sel_stride - 1);
  p.part_f16 = pl.split_len == 32 * 4 && n_cols < 16 && pl.n_splits >= PA_F16_PARTIALS_MIN_SPLITS;   // (as plan_f16_partials)
  PaTiming tm;
  if ((rc = prof_pair(ctx, &tm))) return rc;
  HIPCHK(ctx, pa_launch_decode_gather(p, c.head_dim, ctx->stream, &tm));
  HIPCHK(ctx, pa_launch_combine(p, c.head_dim, ctx->stream));
  return PA_OK;
}

// ---- checkpoint slots ---------------------------------------------------------------------------------
// Device-side copies of the rows written so far (the reference's saveSlot / loadSlot / dropSlot:
// engine/dense.js:20-47, engine/qwen35.js:190-230) and their host form (exportSlot / importState parts:
// engine/qwen35.js:121-131, :151-190): per layer one K part and one V part of pos * kvDim f16, position-major.

static void slot_free(pa_slot& sl) {
  for (int w = 0; w < 4; w++) { for (auto p : sl.t[w]) if (p) (void)hipFree(p); sl.t[w].clear(); }
  sl.pos = 0;
}

// a slot with room for rows [0, pos) of every allocated layer (contents undefined)
static int slot_make(pa_ctx* ctx, const char* who, uint32_t slot, uint32_t pos) {
  if (pos > ctx->cfg.max_seq) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": pos exceeds max_seq");
  auto it = ctx->slots.find(slot);
  if (it != ctx->slots.end() && it->second.pos == pos && it->second.t[0].size() == ctx->layers.size()) {
    bool same = true;                                   // same shape: the buffers are reused (the stream orders the copies)
    for (size_t l = 0; l < ctx->layers.size(); l++) same = same && ((ctx->layers[l].k != nullptr && pos != 0) == (it->second.t[0][l] != nullptr));
    if (same) return PA_OK;
  }
  if (it != ctx->slots.end()) {
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));     // copies out of the old buffers may still be queued
    slot_free(it->second); ctx->slots.erase(it);
  }
  pa_slot sl; sl.pos = pos;
  for (int w = 0; w < 4; w++) sl.t[w].assign(ctx->layers.size(), nullptr);
  for (size_t l = 0; l < ctx->layers.size() && pos; l++) {
    if (!ctx->layers[l].k) continue;
    for (int w = 0; w < n_tensors(ctx); w++) {
      hipError_t e = hipMalloc(&sl.t[w][l], (size_t)pos * ctx->cfg.n_kv_heads * head_row_bytes(ctx, w));
      if (e != hipSuccess) { slot_free(sl); return fail_hip(ctx, e, "slot allocation"); }
    }
  }
  ctx->slots[slot] = std::move(sl);
  return PA_OK;
}

// rows [0, pos) of one tensor between the cache ([nKV][max_seq + 32][hd]) and a slot ([nKV][pos][hd]): one pitched copy
static hipError_t slot_copy(const pa_ctx* ctx, int which, void* cache, void* slot_buf, uint32_t pos, bool to_slot) {
  const size_t plane = (size_t)pos * head_row_bytes(ctx, which), cache_pitch = ((size_t)ctx->cfg.max_seq + 32) * head_row_bytes(ctx, which);
  return to_slot ? hipMemcpy2DAsync(slot_buf, plane, cache, cache_pitch, plane, ctx->cfg.n_kv_heads, hipMemcpyDeviceToDevice, ctx->stream)
                 : hipMemcpy2DAsync(cache, cache_pitch, slot_buf, plane, plane, ctx->cfg.n_kv_heads, hipMemcpyDeviceToDevice, ctx->stream);
}

extern "C" int pa_slot_save(pa_ctx* ctx, uint32_t slot, uint32_t pos) {
  if (!ctx) return PA_ERR_INVALID;
  int rc = slot_make(ctx, "pa_slot_save", slot, pos);
  if (rc) return rc;
  pa_slot& sl = ctx->slots[slot];
  for (size_t l = 0; l < ctx->layers.size(); l++) {
    if (!sl.t[0][l]) continue;
    for (int w = 0; w < n_tensors(ctx); w++) HIPCHK(ctx, slot_copy(ctx, w, ctx->layers[l].tensor(w), sl.t[w][l], pos, true));
  }
  return PA_OK;
}

extern "C" int pa_slot_load(pa_ctx* ctx, uint32_t slot, uint32_t* pos) {
  if (!ctx || !pos) return PA_ERR_INVALID;
  auto it = ctx->slots.find(slot);
  if (it == ctx->slots.end()) return fail(ctx, PA_ERR_INVALID, "pa_slot_load: no saved slot " + std::to_string(slot));
  pa_slot& sl = it->second;
  for (size_t l = 0; l < ctx->layers.size(); l++) {
    if (l >= sl.t[0].size() || !sl.t[0][l]) continue;
    if (!ctx->layers[l].k) return fail(ctx, PA_ERR_INVALID, "pa_slot_load: the slot holds a layer that has no cache now");
    for (int w = 0; w < n_tensors(ctx); w++) HIPCHK(ctx, slot_copy(ctx, w, ctx->layers[l].tensor(w), sl.t[w][l], sl.pos, false));
  }
  *pos = sl.pos;
  return PA_OK;
}

extern "C" int pa_slot_drop(pa_ctx* ctx, uint32_t slot) {
  if (!ctx) return PA_ERR_INVALID;
  auto it = ctx->slots.find(slot);
  if (it == ctx->slots.end()) return PA_OK;               // as dropSlot: dropping an unknown slot is not an error
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  slot_free(it->second); ctx->slots.erase(it);
  return PA_OK;
}

extern "C" int pa_slot_pos(pa_ctx* ctx, uint32_t slot, uint32_t* pos) {
  if (!ctx || !pos) return PA_ERR_INVALID;
  auto it = ctx->slots.find(slot);
  if (it == ctx->slots.end()) return fail(ctx, PA_ERR_INVALID, "pa_slot_pos: no saved slot " + std::to_string(slot));
  *pos = it->second.pos;
  return PA_OK;
}

extern "C" int pa_slot_create(pa_ctx* ctx, uint32_t slot, uint32_t pos) {
  if (!ctx) return PA_ERR_INVALID;
  return slot_make(ctx, "pa_slot_create", slot, pos);
}

// one part between a slot and the host, position-major [pos][nKV * hd] on the host side
static int slot_part(pa_ctx* ctx, const char* who, uint32_t slot, uint32_t layer, int which, void* host, bool to_host) {
  auto it = ctx->slots.find(slot);
  if (it == ctx->slots.end()) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": no saved slot " + std::to_string(slot));
  pa_slot& sl = it->second;
  if (which < 0 || which >= n_tensors(ctx)) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": which must be 0 (K) or 1 (V), or 2 / 3 (their scales) on an int8 cache");
  if (sl.pos == 0) return PA_OK;
  if (layer >= sl.t[0].size() || !sl.t[0][layer]) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": the slot has no such layer");
  if (!host) return fail(ctx, PA_ERR_INVALID, std::string(who) + ": null host buffer");
  const pa_config& c = ctx->cfg;
  const size_t hd_bytes = head_row_bytes(ctx, which), host_pitch = hd_bytes * c.n_kv_heads, plane_bytes = (size_t)sl.pos * hd_bytes;
  unsigned char* dev = (unsigned char*)sl.t[which][layer];
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  std::vector<unsigned char> plane(plane_bytes);
  for (uint32_t g = 0; g < c.n_kv_heads; g++) {
    unsigned char* h = (unsigned char*)host + (size_t)g * hd_bytes;
    if (to_host) {
      HIPCHK(ctx, hipMemcpy(plane.data(), dev + g * plane_bytes, plane_bytes, hipMemcpyDeviceToHost));
      for (uint32_t r = 0; r < sl.pos; r++) memcpy(h + (size_t)r * host_pitch, plane.data() + (size_t)r * hd_bytes, hd_bytes);
    } else {
      for (uint32_t r = 0; r < sl.pos; r++) memcpy(plane.data() + (size_t)r * hd_bytes, h + (size_t)r * host_pitch, hd_bytes);
      HIPCHK(ctx, hipMemcpy(dev + g * plane_bytes, plane.data(), plane_bytes, hipMemcpyHostToDevice));
    }
  }
  return PA_OK;
}
extern "C" int pa_slot_export(pa_ctx* ctx, uint32_t slot, uint32_t layer, int which, void* h_dst) {
  if (!ctx) return PA_ERR_INVALID;
  return slot_part(ctx, "pa_slot_export", slot, layer, which, h_dst, true);
}
extern "C" int pa_slot_import(pa_ctx* ctx, uint32_t slot, uint32_t layer, int which, const void* h_src) {
  if (!ctx) return PA_ERR_INVALID;
  return slot_part(ctx, "pa_slot_import", slot, layer, which, const_cast<void*>(h_src), false);
}

extern "C" const void* pa_kv_device_ptr(pa_ctx* ctx, uint32_t layer, int which) {
  if (!ctx || layer >= ctx->cfg.n_layers) return nullptr;
  return which >= 0 && which < 4 ? (const void*)ctx->layers[layer].tensor(which) : nullptr;
}

// ---- timing -----------------------------------------------------------------------------------------

extern "C" int pa_timer_start(pa_ctx* ctx) {
  if (!ctx) return PA_ERR_INVALID;
  HIPCHK(ctx, hipEventRecord(ctx->t0, ctx->stream));
  return PA_OK;
}
extern "C" int pa_timer_stop(pa_ctx* ctx, float* ms) {
  if (!ctx || !ms) return PA_ERR_INVALID;
  HIPCHK(ctx, hipEventRecord(ctx->t1, ctx->stream));
  HIPCHK(ctx, hipEventSynchronize(ctx->t1));
  HIPCHK(ctx, hipEventElapsedTime(ms, ctx->t0, ctx->t1));
  return PA_OK;
}
extern "C" int pa_profile_enable(pa_ctx* ctx, int on) {
  if (!ctx) return PA_ERR_INVALID;
  ctx->profiling = on != 0;
  ctx->prof_used = 0; ctx->prof_aux_used = 0;
  return PA_OK;
}
extern "C" int pa_profile_read(pa_ctx* ctx, float* ms_sum, uint32_t* count) {
  if (!ctx || !ms_sum || !count) return PA_ERR_INVALID;
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  float sum = 0.f;
  for (size_t i = 0; i + 1 < ctx->prof_used; i += 2) {
    float ms = 0.f;
    HIPCHK(ctx, hipEventElapsedTime(&ms, ctx->prof_events[i], ctx->prof_events[i + 1]));
    sum += ms;
  }
  *ms_sum = sum; *count = (uint32_t)(ctx->prof_used / 2);
  ctx->prof_used = 0; ctx->prof_aux_used = 0;
  return PA_OK;
}
extern "C" int pa_profile_read_each(pa_ctx* ctx, float* ms, uint32_t cap, uint32_t* count) {
  if (!ctx || !count || (!ms && cap)) return PA_ERR_INVALID;
  HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
  const size_t n = ctx->prof_used / 2;
  for (size_t i = 0; i < n && i < cap; i++) HIPCHK(ctx, hipEventElapsedTime(&ms[i], ctx->prof_events[2 * i], ctx->prof_events[2 * i + 1]));
  *count = (uint32_t)n;
  ctx->prof_used = 0; ctx->prof_aux_used = 0;
  return PA_OK;
}
