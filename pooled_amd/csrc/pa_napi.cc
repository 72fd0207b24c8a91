// Thin Node-API layer over the C ABI of include/pooled_attn.h.
//
// pooled already runs its engines in Node on a WebGPU addon (packages/room-node/index.js:1-3,
// cli/lib/dawn.js:1-13); this addon is what sits under the JavaScript host shim instead of that WebGPU device
// for the attention path.  Every export maps 1:1 to a pa_* function: numbers in, numbers out; device addresses
// travel as JS numbers (GPU virtual addresses fit in 53 bits); host data as TypedArrays.  A non-zero status
// becomes a thrown Error carrying pa_last_error().  No logic lives here.
#include <node_api.h>
#include <stdint.h>
#include <string.h>
#include <string>
#include "pooled_attn.h"

#define NAPI_OK(call) do { if ((call) != napi_ok) { napi_throw_error(env, nullptr, "pooled_attn addon: N-API call failed: " #call); return nullptr; } } while (0)

static napi_value throw_pa(napi_env env, pa_ctx* ctx, int rc, const char* who) {
  std::string msg = std::string(who) + " failed (" + std::to_string(rc) + "): " + pa_last_error(ctx);
  napi_value code, err, text;
  napi_create_string_utf8(env, rc == PA_ERR_UNSUPPORTED ? "PA_ERR_UNSUPPORTED" : rc == PA_ERR_INVALID ? "PA_ERR_INVALID" : rc == PA_ERR_NOMEM ? "PA_ERR_NOMEM" : "PA_ERR_HIP", NAPI_AUTO_LENGTH, &code);
  napi_create_string_utf8(env, msg.c_str(), NAPI_AUTO_LENGTH, &text);
  napi_create_error(env, code, text, &err);
  napi_throw(env, err);
  return nullptr;
}

// What the JS handle points at.  destroy() clears ctx, so a stale handle is refused instead of reaching freed memory;
// the box itself lives until the handle is garbage collected.
struct CtxBox { pa_ctx* ctx; };
static void box_finalize(napi_env, void* data, void*) { CtxBox* b = (CtxBox*)data; if (b) { if (b->ctx) pa_destroy(b->ctx); delete b; } }

struct Args {
  napi_env env; size_t argc; napi_value argv[16]; bool ok;
  Args(napi_env e, napi_callback_info info) : env(e), argc(16), ok(true) { if (napi_get_cb_info(e, info, &argc, argv, nullptr, nullptr) != napi_ok) ok = false; }
  double num(size_t i) { double d = 0; if (i >= argc || napi_get_value_double(env, argv[i], &d) != napi_ok) ok = false; return d; }
  uint32_t u32(size_t i) { return (uint32_t)num(i); }
  void* ptr(size_t i) {                       // device address as a number; null / undefined -> nullptr
    if (i >= argc) return nullptr;
    napi_valuetype t; napi_typeof(env, argv[i], &t);
    if (t == napi_null || t == napi_undefined) return nullptr;
    return (void*)(uintptr_t)num(i);
  }
  // the handle create() returned: an external holding a CtxBox; a destroyed context reads as a bad argument
  pa_ctx* ctx(size_t i) {
    void* p = nullptr;
    if (i >= argc || napi_get_value_external(env, argv[i], &p) != napi_ok || !p || !((CtxBox*)p)->ctx) { ok = false; return nullptr; }
    return ((CtxBox*)p)->ctx;
  }
  CtxBox* box(size_t i) { void* p = nullptr; if (i >= argc || napi_get_value_external(env, argv[i], &p) != napi_ok) ok = false; return (CtxBox*)p; }
  void* host(size_t i, size_t* bytes) {       // TypedArray / ArrayBuffer contents
    void* data = nullptr; *bytes = 0;
    bool is = false;
    if (i < argc && napi_is_typedarray(env, argv[i], &is) == napi_ok && is) {
      napi_typedarray_type ty; size_t len; napi_value ab; size_t off;
      if (napi_get_typedarray_info(env, argv[i], &ty, &len, &data, &ab, &off) != napi_ok) ok = false;
      static const size_t esz[] = {1, 1, 1, 2, 2, 4, 4, 4, 8, 8, 8};
      *bytes = len * esz[ty];
      return data;
    }
    if (i < argc && napi_is_arraybuffer(env, argv[i], &is) == napi_ok && is) { if (napi_get_arraybuffer_info(env, argv[i], &data, bytes) != napi_ok) ok = false; return data; }
    ok = false; return nullptr;
  }
};
#define ARGS Args a(env, info)
#define CHECK_ARGS(who) do { if (!a.ok) { napi_throw_type_error(env, nullptr, who ": bad arguments"); return nullptr; } } while (0)

static napi_value num_value(napi_env env, double d) { napi_value v; napi_create_double(env, d, &v); return v; }
static napi_value undefined(napi_env env) { napi_value v; napi_get_undefined(env, &v); return v; }

static uint32_t prop_u32(napi_env env, napi_value o, const char* k, uint32_t def) {
  napi_value v; bool has = false;
  if (napi_has_named_property(env, o, k, &has) != napi_ok || !has) return def;
  double d; if (napi_get_named_property(env, o, k, &v) != napi_ok || napi_get_value_double(env, v, &d) != napi_ok) return def;
  return (uint32_t)d;
}
static double prop_f64(napi_env env, napi_value o, const char* k, double def) {
  napi_value v; bool has = false;
  if (napi_has_named_property(env, o, k, &has) != napi_ok || !has) return def;
  double d; if (napi_get_named_property(env, o, k, &v) != napi_ok || napi_get_value_double(env, v, &d) != napi_ok) return def;
  return d;
}

// create({nH, nKV, hd, nRot, ropeTheta, eps, maxSeq, nLayers, maxCols, flags}) -> handle
static napi_value Create(napi_env env, napi_callback_info info) {
  ARGS;
  if (a.argc < 1) { napi_throw_type_error(env, nullptr, "create: config object expected"); return nullptr; }
  napi_value o = a.argv[0];
  pa_config c; memset(&c, 0, sizeof c);
  c.n_heads = prop_u32(env, o, "nH", 0); c.n_kv_heads = prop_u32(env, o, "nKV", 0); c.head_dim = prop_u32(env, o, "hd", 0);
  c.n_rot = prop_u32(env, o, "nRot", c.head_dim); c.rope_theta = (float)prop_f64(env, o, "ropeTheta", 1e6); c.eps = (float)prop_f64(env, o, "eps", 1e-6);
  c.max_seq = prop_u32(env, o, "maxSeq", 0); c.n_layers = prop_u32(env, o, "nLayers", 1); c.max_cols = prop_u32(env, o, "maxCols", 16);
  c.flags = prop_u32(env, o, "flags", PA_FLAG_QK_NORM);
  pa_ctx* ctx = nullptr;
  int rc = pa_create(&c, &ctx);
  if (rc) return throw_pa(env, nullptr, rc, "pa_create");
  CtxBox* box = new CtxBox{ctx};
  napi_value ext;
  if (napi_create_external(env, box, box_finalize, nullptr, &ext) != napi_ok) { pa_destroy(ctx); delete box; napi_throw_error(env, nullptr, "pooled_attn addon: napi_create_external failed"); return nullptr; }
  return ext;
}
static napi_value Destroy(napi_env env, napi_callback_info info) {
  ARGS; CtxBox* b = a.box(0); CHECK_ARGS("destroy");
  if (b && b->ctx) { pa_destroy(b->ctx); b->ctx = nullptr; }
  return undefined(env);
}
static napi_value LastError(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.argc ? a.ctx(0) : nullptr; a.ok = true; napi_value v; napi_create_string_utf8(env, pa_last_error(c), NAPI_AUTO_LENGTH, &v); return v; }
static napi_value Version(napi_env env, napi_callback_info) { napi_value v; napi_create_string_utf8(env, pa_version(), NAPI_AUTO_LENGTH, &v); return v; }

static napi_value LayerAlloc(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); uint32_t l = a.u32(1); CHECK_ARGS("layerAlloc"); int rc = pa_layer_alloc(c, l); if (rc) return throw_pa(env, c, rc, "pa_layer_alloc"); return undefined(env); }
static napi_value Sync(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); CHECK_ARGS("sync"); int rc = pa_sync(c); if (rc) return throw_pa(env, c, rc, "pa_sync"); return undefined(env); }
static napi_value SetStream(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); void* s = a.ptr(1); CHECK_ARGS("setStream"); int rc = pa_set_stream(c, s); if (rc) return throw_pa(env, c, rc, "pa_set_stream"); return undefined(env); }
static napi_value Malloc(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); double n = a.num(1); CHECK_ARGS("malloc"); void* p = nullptr; int rc = pa_malloc(c, (size_t)n, &p); if (rc) return throw_pa(env, c, rc, "pa_malloc"); return num_value(env, (double)(uintptr_t)p); }
static napi_value Free(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); void* p = a.ptr(1); CHECK_ARGS("free"); int rc = pa_free(c, p); if (rc) return throw_pa(env, c, rc, "pa_free"); return undefined(env); }
// upload(ctx, dPtr, typedArray [, byteOffsetOnDevice])
static napi_value Upload(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); char* d = (char*)a.ptr(1); size_t n; void* h = a.host(2, &n); size_t off = a.argc > 3 ? (size_t)a.num(3) : 0; CHECK_ARGS("upload");
  int rc = pa_upload(c, d + off, h, n); if (rc) return throw_pa(env, c, rc, "pa_upload"); return undefined(env);
}
static napi_value Download(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); size_t n; void* h = a.host(1, &n); const char* d = (const char*)a.ptr(2); size_t off = a.argc > 3 ? (size_t)a.num(3) : 0; CHECK_ARGS("download");
  int rc = pa_download(c, h, d + off, n); if (rc) return throw_pa(env, c, rc, "pa_download"); return undefined(env);
}
// glueKv(ctx, layer, dQ, qStride, dK, kStride, dV, vStride, dQw, dKw, basePos, nCols)
static napi_value GlueKv(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0);
  uint32_t layer = a.u32(1); const float* q = (const float*)a.ptr(2); uint32_t qs = a.u32(3); const float* k = (const float*)a.ptr(4); uint32_t ks = a.u32(5);
  const float* v = (const float*)a.ptr(6); uint32_t vs = a.u32(7); const float* qw = (const float*)a.ptr(8); const float* kw = (const float*)a.ptr(9);
  uint32_t base = a.u32(10), n = a.u32(11); CHECK_ARGS("glueKv");
  int rc = pa_glue_kv(c, layer, q, qs, k, ks, v, vs, qw, kw, base, n); if (rc) return throw_pa(env, c, rc, "pa_glue_kv"); return undefined(env);
}
// glue(ctx, dQ, qStride, dK, kStride, dQw, dKw, basePos, nCols)
static napi_value Glue(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0);
  const float* q = (const float*)a.ptr(1); uint32_t qs = a.u32(2); float* k = (float*)a.ptr(3); uint32_t ks = a.u32(4);
  const float* qw = (const float*)a.ptr(5); const float* kw = (const float*)a.ptr(6); uint32_t base = a.u32(7), n = a.u32(8); CHECK_ARGS("glue");
  int rc = pa_glue(c, q, qs, k, ks, qw, kw, base, n); if (rc) return throw_pa(env, c, rc, "pa_glue"); return undefined(env);
}
// kvStore(ctx, layer, dK, kStride, dV, vStride, basePos, nCols)
static napi_value KvStore(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0);
  uint32_t layer = a.u32(1); const float* k = (const float*)a.ptr(2); uint32_t ks = a.u32(3); const float* v = (const float*)a.ptr(4); uint32_t vs = a.u32(5);
  uint32_t base = a.u32(6), n = a.u32(7); CHECK_ARGS("kvStore");
  int rc = pa_kv_store(c, layer, k, ks, v, vs, base, n); if (rc) return throw_pa(env, c, rc, "pa_kv_store"); return undefined(env);
}
static napi_value QBuffer(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); CHECK_ARGS("qBuffer"); return num_value(env, (double)(uintptr_t)pa_q_buffer(c)); }
static napi_value GateBuffer(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); CHECK_ARGS("gateBuffer"); return num_value(env, (double)(uintptr_t)pa_gate_buffer(c)); }
// attn(ctx, kind, layer, dQ|null, qStride, dGate|null, gateStride, basePos, nCols, dOut, outStride, outDtype)
static napi_value Attn(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0);
  uint32_t kind = a.u32(1), layer = a.u32(2); const float* q = (const float*)a.ptr(3); uint32_t qs = a.u32(4);
  const float* g = (const float*)a.ptr(5); uint32_t gs = a.u32(6); uint32_t base = a.u32(7), n = a.u32(8);
  void* out = a.ptr(9); uint32_t os = a.u32(10); int dt = (int)a.u32(11); CHECK_ARGS("attn");
  int rc = kind == 0 ? pa_attn_decode(c, layer, q, qs, g, gs, base, n, out, os, dt) : pa_attn_prefill(c, layer, q, qs, g, gs, base, n, out, os, dt);
  if (rc) return throw_pa(env, c, rc, kind == 0 ? "pa_attn_decode" : "pa_attn_prefill");
  return undefined(env);
}
// attnDecodeStep(ctx, layer, qIn, k, v, qw|null, kw|null, pos, out, outDtype): the fused one-token block
static napi_value AttnDecodeStep(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0);
  uint32_t layer = a.u32(1); const float* q = (const float*)a.ptr(2); const float* k = (const float*)a.ptr(3); const float* v = (const float*)a.ptr(4);
  const float* qw = (const float*)a.ptr(5); const float* kw = (const float*)a.ptr(6); uint32_t pos = a.u32(7);
  void* out = a.ptr(8); int dt = (int)a.u32(9); CHECK_ARGS("attnDecodeStep");
  int rc = pa_attn_decode_step(c, layer, q, k, v, qw, kw, pos, out, dt);
  if (rc) return throw_pa(env, c, rc, "pa_attn_decode_step");
  return undefined(env);
}
// copyD2d(ctx, dst, src, bytes): device-to-device copy on the context's stream
static napi_value CopyD2d(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); void* dst = a.ptr(1); const void* src = a.ptr(2); size_t n = (size_t)a.num(3); CHECK_ARGS("copyD2d");
  int rc = pa_copy_d2d(c, dst, src, n); if (rc) return throw_pa(env, c, rc, "pa_copy_d2d"); return undefined(env);
}
// attnGather(ctx, layer, q|null, qStride, gate|null, gateStride, sel, selStride, maxRows, nCols, out, outStride, outDtype)
static napi_value AttnGather(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0);
  uint32_t layer = a.u32(1); const float* q = (const float*)a.ptr(2); uint32_t qs = a.u32(3);
  const float* g = (const float*)a.ptr(4); uint32_t gs = a.u32(5); const uint32_t* sel = (const uint32_t*)a.ptr(6);
  uint32_t ss = a.u32(7), mr = a.u32(8), n = a.u32(9); void* out = a.ptr(10); uint32_t os = a.u32(11); int dt = (int)a.u32(12); CHECK_ARGS("attnGather");
  int rc = pa_attn_decode_gather(c, layer, q, qs, g, gs, sel, ss, mr, n, out, os, dt);
  if (rc) return throw_pa(env, c, rc, "pa_attn_decode_gather");
  return undefined(env);
}
// planQuery(ctx, kind, basePos, nCols) -> {kernel, splitLen, nSplits, colGroups, colsPerGroup, waves, rowBlocks, slots}
static napi_value PlanQuery(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); int kind = (int)a.u32(1); uint32_t base = a.u32(2), n = a.u32(3); CHECK_ARGS("planQuery");
  pa_plan pl; int rc = pa_plan_query(c, kind, base, n, &pl); if (rc) return throw_pa(env, c, rc, "pa_plan_query");
  napi_value o; NAPI_OK(napi_create_object(env, &o));
  const char* names[] = {"kernel", "splitLen", "nSplits", "colGroups", "colsPerGroup", "waves", "rowBlocks", "slots"};
  const uint32_t vals[] = {pl.kernel, pl.split_len, pl.n_splits, pl.col_groups, pl.cols_per_group, pl.waves, pl.row_blocks, pl.slots};
  for (int i = 0; i < 8; i++) napi_set_named_property(env, o, names[i], num_value(env, vals[i]));
  return o;
}
static napi_value SetPrefillTile(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); int m = (int)a.u32(1); CHECK_ARGS("setPrefillTile"); int rc = pa_set_prefill_tile(c, m); if (rc) return throw_pa(env, c, rc, "pa_set_prefill_tile"); return undefined(env); }
static napi_value SetWeightCache(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); double b = a.num(1); CHECK_ARGS("setWeightCache"); int rc = pa_set_weight_cache(c, b <= 0 ? 0 : (size_t)b); if (rc) return throw_pa(env, c, rc, "pa_set_weight_cache"); return undefined(env); }
static napi_value SetDecodeSplits(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); uint32_t s = a.u32(1); CHECK_ARGS("setDecodeSplits"); int rc = pa_set_decode_splits(c, s); if (rc) return throw_pa(env, c, rc, "pa_set_decode_splits"); return undefined(env); }
// kvRead(ctx, layer, which, row0, nRows, Uint16Array) / kvWrite(ctx, layer, which, row0, nRows, Uint16Array)
static napi_value KvRead(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); uint32_t layer = a.u32(1); int which = (int)a.u32(2); uint32_t r0 = a.u32(3), nr = a.u32(4); size_t n; void* h = a.host(5, &n); CHECK_ARGS("kvRead");
  if (n < (size_t)nr * pa_kv_row_bytes(c, which)) { napi_throw_range_error(env, nullptr, "kvRead: array shorter than nRows rows of this cache tensor"); return nullptr; }
  int rc = pa_kv_read(c, layer, which, r0, nr, h); if (rc) return throw_pa(env, c, rc, "pa_kv_read"); return undefined(env);
}
static napi_value KvWrite(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); uint32_t layer = a.u32(1); int which = (int)a.u32(2); uint32_t r0 = a.u32(3), nr = a.u32(4); size_t n; void* h = a.host(5, &n); CHECK_ARGS("kvWrite");
  if (n < (size_t)nr * pa_kv_row_bytes(c, which)) { napi_throw_range_error(env, nullptr, "kvWrite: array shorter than nRows rows of this cache tensor"); return nullptr; }
  int rc = pa_kv_write(c, layer, which, r0, nr, h); if (rc) return throw_pa(env, c, rc, "pa_kv_write"); return undefined(env);
}
static napi_value KvDevicePtr(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); uint32_t layer = a.u32(1); int which = (int)a.u32(2); CHECK_ARGS("kvDevicePtr"); return num_value(env, (double)(uintptr_t)pa_kv_device_ptr(c, layer, which)); }
static napi_value TimerStart(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); CHECK_ARGS("timerStart"); int rc = pa_timer_start(c); if (rc) return throw_pa(env, c, rc, "pa_timer_start"); return undefined(env); }
static napi_value TimerStop(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); CHECK_ARGS("timerStop"); float ms = 0; int rc = pa_timer_stop(c, &ms); if (rc) return throw_pa(env, c, rc, "pa_timer_stop"); return num_value(env, ms); }
static napi_value ProfileEnable(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); int on = (int)a.u32(1); CHECK_ARGS("profileEnable"); int rc = pa_profile_enable(c, on); if (rc) return throw_pa(env, c, rc, "pa_profile_enable"); return undefined(env); }
static napi_value ProfileRead(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); CHECK_ARGS("profileRead"); float ms = 0; uint32_t n = 0; int rc = pa_profile_read(c, &ms, &n); if (rc) return throw_pa(env, c, rc, "pa_profile_read");
  napi_value o; NAPI_OK(napi_create_object(env, &o)); napi_set_named_property(env, o, "ms", num_value(env, ms)); napi_set_named_property(env, o, "count", num_value(env, n)); return o;
}

// ---- checkpoint slots: slotSave(ctx, id, pos), slotLoad(ctx, id) -> pos, slotDrop(ctx, id), slotPos(ctx, id) -> pos,
//      slotCreate(ctx, id, pos), slotExport(ctx, id, layer, which, Uint16Array), slotImport(ctx, id, layer, which, Uint16Array)
static napi_value SlotSave(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); uint32_t id = a.u32(1), pos = a.u32(2); CHECK_ARGS("slotSave"); int rc = pa_slot_save(c, id, pos); if (rc) return throw_pa(env, c, rc, "pa_slot_save"); return undefined(env); }
static napi_value SlotLoad(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); uint32_t id = a.u32(1); CHECK_ARGS("slotLoad"); uint32_t pos = 0; int rc = pa_slot_load(c, id, &pos); if (rc) return throw_pa(env, c, rc, "pa_slot_load"); return num_value(env, pos); }
static napi_value SlotDrop(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); uint32_t id = a.u32(1); CHECK_ARGS("slotDrop"); int rc = pa_slot_drop(c, id); if (rc) return throw_pa(env, c, rc, "pa_slot_drop"); return undefined(env); }
static napi_value SlotPos(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); uint32_t id = a.u32(1); CHECK_ARGS("slotPos"); uint32_t pos = 0; int rc = pa_slot_pos(c, id, &pos); if (rc) return throw_pa(env, c, rc, "pa_slot_pos"); return num_value(env, pos); }
static napi_value SlotCreate(napi_env env, napi_callback_info info) { ARGS; pa_ctx* c = a.ctx(0); uint32_t id = a.u32(1), pos = a.u32(2); CHECK_ARGS("slotCreate"); int rc = pa_slot_create(c, id, pos); if (rc) return throw_pa(env, c, rc, "pa_slot_create"); return undefined(env); }
static napi_value SlotExport(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); uint32_t id = a.u32(1), layer = a.u32(2); int which = (int)a.u32(3); size_t n; void* h = a.host(4, &n); CHECK_ARGS("slotExport");
  { uint32_t pos = 0; int rc0 = pa_slot_pos(c, id, &pos); if (rc0) return throw_pa(env, c, rc0, "pa_slot_pos");
    if (n < (size_t)pos * pa_kv_row_bytes(c, which)) { napi_throw_range_error(env, nullptr, "slotExport: array shorter than the slot's rows of this cache tensor"); return nullptr; } }
  int rc = pa_slot_export(c, id, layer, which, h); if (rc) return throw_pa(env, c, rc, "pa_slot_export"); return undefined(env);
}
static napi_value SlotImport(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); uint32_t id = a.u32(1), layer = a.u32(2); int which = (int)a.u32(3); size_t n; void* h = a.host(4, &n); CHECK_ARGS("slotImport");
  { uint32_t pos = 0; int rc0 = pa_slot_pos(c, id, &pos); if (rc0) return throw_pa(env, c, rc0, "pa_slot_pos");
    if (n < (size_t)pos * pa_kv_row_bytes(c, which)) { napi_throw_range_error(env, nullptr, "slotImport: array shorter than the slot's rows of this cache tensor"); return nullptr; } }
  int rc = pa_slot_import(c, id, layer, which, h); if (rc) return throw_pa(env, c, rc, "pa_slot_import"); return undefined(env);
}

// ---- projections (one-token passes) ----
// weightCreate(ctx, kind, dOut, dIn, valuesTypedArray, scalesUint16Array | null) -> weight handle (a number)
static napi_value WeightCreate(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); int kind = (int)a.u32(1); uint32_t d_out = a.u32(2), d_in = a.u32(3);
  size_t nw = 0, ns = 0; void* hw = a.host(4, &nw);
  void* hs = nullptr;
  if (a.argc > 5) { napi_valuetype t; napi_typeof(env, a.argv[5], &t); if (t != napi_null && t != napi_undefined) hs = a.host(5, &ns); }
  CHECK_ARGS("weightCreate");
  const size_t want_w = kind == PA_W_F32 ? (size_t)d_out * d_in * 4 : kind == PA_W_Q8_0 ? (size_t)d_out * d_in : (size_t)d_out * d_in / 2;
  const size_t want_s = kind == PA_W_F32 ? 0 : (size_t)d_out * (d_in / 32) * 2;
  if (nw < want_w || (want_s && ns < want_s)) { napi_throw_range_error(env, nullptr, "weightCreate: plane shorter than dOut x dIn needs"); return nullptr; }
  pa_weight* w = nullptr;
  int rc = pa_weight_create(c, kind, d_out, d_in, hw, hs, &w);
  if (rc) return throw_pa(env, c, rc, "pa_weight_create");
  return num_value(env, (double)(uintptr_t)w);
}
static napi_value WeightDestroy(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); pa_weight* w = (pa_weight*)a.ptr(1); CHECK_ARGS("weightDestroy");
  int rc = pa_weight_destroy(c, w); if (rc) return throw_pa(env, c, rc, "pa_weight_destroy"); return undefined(env);
}
// gemv(ctx, weight, x, y, acc)
static napi_value Gemv(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); pa_weight* w = (pa_weight*)a.ptr(1); const float* x = (const float*)a.ptr(2); float* y = (float*)a.ptr(3); int acc = (int)a.u32(4);
  CHECK_ARGS("gemv");
  int rc = pa_gemv(c, w, x, y, acc); if (rc) return throw_pa(env, c, rc, "pa_gemv"); return undefined(env);
}
// gemvNorm(ctx, weight, xRaw, normW, xnOut | null, y)
static napi_value GemvNorm(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); pa_weight* w = (pa_weight*)a.ptr(1); const float* x = (const float*)a.ptr(2); const float* nw = (const float*)a.ptr(3);
  float* xn = (float*)a.ptr(4); float* y = (float*)a.ptr(5); CHECK_ARGS("gemvNorm");
  int rc = pa_gemv_norm(c, w, x, nw, xn, y); if (rc) return throw_pa(env, c, rc, "pa_gemv_norm"); return undefined(env);
}
// attnLayerDecode(ctx, layer, wQkv, wO, attnNormW, qNormW, kNormW, x, pos)
static napi_value AttnLayerDecode(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); uint32_t layer = a.u32(1); pa_weight* wqkv = (pa_weight*)a.ptr(2); pa_weight* wo = (pa_weight*)a.ptr(3);
  const float* nw = (const float*)a.ptr(4); const float* qw = (const float*)a.ptr(5); const float* kw = (const float*)a.ptr(6);
  float* x = (float*)a.ptr(7); uint32_t pos = a.u32(8); CHECK_ARGS("attnLayerDecode");
  int rc = pa_attn_layer_decode(c, layer, wqkv, wo, nw, qw, kw, x, pos); if (rc) return throw_pa(env, c, rc, "pa_attn_layer_decode"); return undefined(env);
}

// rmsnormF16(ctx, x, xStride, normW, dim, nCols, xnF16, xnStride)
static napi_value RmsnormF16(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); const float* x = (const float*)a.ptr(1); uint32_t xs = a.u32(2); const float* nw = (const float*)a.ptr(3);
  uint32_t dim = a.u32(4), n = a.u32(5); void* out = a.ptr(6); uint32_t os = a.u32(7); CHECK_ARGS("rmsnormF16");
  int rc = pa_rmsnorm_f16(c, x, xs, nw, dim, n, out, os); if (rc) return throw_pa(env, c, rc, "pa_rmsnorm_f16"); return undefined(env);
}
// gemm(ctx, weight, xF16, xStride, nCols, y, yStride, acc)
static napi_value Gemm(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); pa_weight* w = (pa_weight*)a.ptr(1); const void* x = a.ptr(2); uint32_t xs = a.u32(3), n = a.u32(4);
  float* y = (float*)a.ptr(5); uint32_t ys = a.u32(6); int acc = (int)a.u32(7); CHECK_ARGS("gemm");
  int rc = pa_gemm(c, w, x, xs, n, y, ys, acc); if (rc) return throw_pa(env, c, rc, "pa_gemm"); return undefined(env);
}
// attnLayerPrefill(ctx, layer, wQkv, wO, attnNormW, qNormW, kNormW, x, xStride, basePos, nCols)
static napi_value AttnLayerPrefill(napi_env env, napi_callback_info info) {
  ARGS; pa_ctx* c = a.ctx(0); uint32_t layer = a.u32(1); pa_weight* wqkv = (pa_weight*)a.ptr(2); pa_weight* wo = (pa_weight*)a.ptr(3);
  const float* nw = (const float*)a.ptr(4); const float* qw = (const float*)a.ptr(5); const float* kw = (const float*)a.ptr(6);
  float* x = (float*)a.ptr(7); uint32_t xs = a.u32(8), base = a.u32(9), n = a.u32(10); CHECK_ARGS("attnLayerPrefill");
  int rc = pa_attn_layer_prefill(c, layer, wqkv, wo, nw, qw, kw, x, xs, base, n); if (rc) return throw_pa(env, c, rc, "pa_attn_layer_prefill"); return undefined(env);
}

static napi_value Init(napi_env env, napi_value exports) {
  struct { const char* name; napi_callback fn; } table[] = {
    {"create", Create}, {"destroy", Destroy}, {"lastError", LastError}, {"version", Version}, {"layerAlloc", LayerAlloc}, {"sync", Sync},
    {"setStream", SetStream}, {"malloc", Malloc}, {"free", Free}, {"upload", Upload}, {"download", Download}, {"glueKv", GlueKv}, {"glue", Glue},
    {"kvStore", KvStore}, {"qBuffer", QBuffer}, {"gateBuffer", GateBuffer}, {"attn", Attn}, {"planQuery", PlanQuery},
    {"setDecodeSplits", SetDecodeSplits}, {"setPrefillTile", SetPrefillTile}, {"setWeightCache", SetWeightCache}, {"kvRead", KvRead}, {"kvWrite", KvWrite}, {"kvDevicePtr", KvDevicePtr}, {"timerStart", TimerStart},
    {"timerStop", TimerStop}, {"profileEnable", ProfileEnable}, {"profileRead", ProfileRead}, {"attnDecodeStep", AttnDecodeStep},
    {"copyD2d", CopyD2d}, {"attnGather", AttnGather}, {"slotSave", SlotSave}, {"slotLoad", SlotLoad}, {"slotDrop", SlotDrop}, {"slotPos", SlotPos},
    {"slotCreate", SlotCreate}, {"slotExport", SlotExport}, {"slotImport", SlotImport}, {"weightCreate", WeightCreate},
    {"weightDestroy", WeightDestroy}, {"gemv", Gemv}, {"gemvNorm", GemvNorm}, {"attnLayerDecode", AttnLayerDecode},
    {"rmsnormF16", RmsnormF16}, {"gemm", Gemm}, {"attnLayerPrefill", AttnLayerPrefill},
  };
  for (auto& t : table) {
    napi_value fn;
    if (napi_create_function(env, t.name, NAPI_AUTO_LENGTH, t.fn, nullptr, &fn) != napi_ok) return nullptr;
    if (napi_set_named_property(env, exports, t.name, fn) != napi_ok) return nullptr;
  }
  return exports;
}
NAPI_MODULE(pooled_attn, Init)
