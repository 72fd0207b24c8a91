"""ctypes binding of the C ABI in include/pooled_attn.h (used by the tests, smoke and bench).

The product is libpooled_attn.so; this module only loads it and moves numpy arrays in and out of HBM through
the library's own pa_malloc / pa_upload / pa_download.  There is no CPU fallback: if the shared library is
missing, loading raises.
"""
import ctypes
import os
import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libpooled_attn.so")

PA_OK, PA_ERR_INVALID, PA_ERR_UNSUPPORTED, PA_ERR_HIP, PA_ERR_NOMEM = 0, 1, 2, 3, 4
PA_FLAG_QK_NORM, PA_FLAG_GATE, PA_FLAG_KV_Q8, PA_FLAG_VERIFY_EXACT = 1, 2, 4, 8
PA_W_F32, PA_W_Q8_0, PA_W_Q4_0 = 0, 1, 2
PA_OUT_F32, PA_OUT_F16 = 0, 1

u32, c_int, vp, f32p = ctypes.c_uint32, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p


class PaConfig(ctypes.Structure):
    _fields_ = [("n_heads", u32), ("n_kv_heads", u32), ("head_dim", u32), ("n_rot", u32),
                ("rope_theta", ctypes.c_float), ("eps", ctypes.c_float), ("max_seq", u32), ("n_layers", u32),
                ("max_cols", u32), ("flags", u32)]


class PaPlan(ctypes.Structure):
    _fields_ = [(n, u32) for n in ("kernel", "split_len", "n_splits", "col_groups", "cols_per_group", "waves",
                                   "row_blocks", "slots")]


# name -> (restype, argtypes); every symbol include/pooled_attn.h declares
SYMBOLS = {
    "pa_create": (c_int, [ctypes.POINTER(PaConfig), ctypes.POINTER(vp)]),
    "pa_destroy": (c_int, [vp]),
    "pa_last_error": (ctypes.c_char_p, [vp]),
    "pa_layer_alloc": (c_int, [vp, u32]),
    "pa_set_stream": (c_int, [vp, vp]),
    "pa_sync": (c_int, [vp]),
    "pa_malloc": (c_int, [vp, ctypes.c_size_t, ctypes.POINTER(vp)]),
    "pa_free": (c_int, [vp, vp]),
    "pa_upload": (c_int, [vp, vp, vp, ctypes.c_size_t]),
    "pa_download": (c_int, [vp, vp, vp, ctypes.c_size_t]),
    "pa_copy_d2d": (c_int, [vp, vp, vp, ctypes.c_size_t]),
    "pa_glue_kv": (c_int, [vp, u32, f32p, u32, f32p, u32, f32p, u32, f32p, f32p, u32, u32]),
    "pa_glue": (c_int, [vp, f32p, u32, f32p, u32, f32p, f32p, u32, u32]),
    "pa_kv_store": (c_int, [vp, u32, f32p, u32, f32p, u32, u32, u32]),
    "pa_q_buffer": (vp, [vp]),
    "pa_gate_buffer": (vp, [vp]),
    "pa_attn_decode": (c_int, [vp, u32, f32p, u32, f32p, u32, u32, u32, vp, u32, c_int]),
    "pa_attn_prefill": (c_int, [vp, u32, f32p, u32, f32p, u32, u32, u32, vp, u32, c_int]),
    "pa_attn_decode_gather": (c_int, [vp, u32, f32p, u32, f32p, u32, vp, u32, u32, u32, vp, u32, c_int]),
    "pa_attn_decode_step": (c_int, [vp, u32, f32p, f32p, f32p, f32p, f32p, u32, vp, c_int]),
    "pa_attn_decode_step_noalloc": (c_int, [vp, u32, f32p, f32p, f32p, f32p, f32p, u32, vp, c_int]),
    "pa_plan_query": (c_int, [vp, c_int, u32, u32, ctypes.POINTER(PaPlan)]),
    "pa_set_decode_splits": (c_int, [vp, u32]),
    "pa_set_prefill_tile": (c_int, [vp, c_int]),
    "pa_set_weight_cache": (c_int, [vp, ctypes.c_size_t]),
    "pa_kv_read": (c_int, [vp, u32, c_int, u32, u32, vp]),
    "pa_kv_write": (c_int, [vp, u32, c_int, u32, u32, vp]),
    "pa_kv_row_bytes": (ctypes.c_size_t, [vp, c_int]),
    "pa_kv_device_ptr": (vp, [vp, u32, c_int]),
    "pa_timer_start": (c_int, [vp]),
    "pa_timer_stop": (c_int, [vp, ctypes.POINTER(ctypes.c_float)]),
    "pa_profile_enable": (c_int, [vp, c_int]),
    "pa_profile_read": (c_int, [vp, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(u32)]),
    "pa_profile_read_each": (c_int, [vp, ctypes.POINTER(ctypes.c_float), u32, ctypes.POINTER(u32)]),
    "pa_slot_save": (c_int, [vp, u32, u32]),
    "pa_slot_load": (c_int, [vp, u32, ctypes.POINTER(u32)]),
    "pa_slot_drop": (c_int, [vp, u32]),
    "pa_slot_pos": (c_int, [vp, u32, ctypes.POINTER(u32)]),
    "pa_slot_create": (c_int, [vp, u32, u32]),
    "pa_slot_export": (c_int, [vp, u32, u32, c_int, vp]),
    "pa_slot_import": (c_int, [vp, u32, u32, c_int, vp]),
    "pa_weight_create": (c_int, [vp, c_int, u32, u32, vp, vp, ctypes.POINTER(vp)]),
    "pa_weight_destroy": (c_int, [vp, vp]),
    "pa_gemv": (c_int, [vp, vp, f32p, f32p, c_int]),
    "pa_gemv_norm": (c_int, [vp, vp, f32p, f32p, f32p, f32p]),
    "pa_attn_layer_decode": (c_int, [vp, u32, vp, vp, f32p, f32p, f32p, f32p, u32]),
    "pa_rmsnorm_f16": (c_int, [vp, f32p, u32, f32p, u32, u32, vp, u32]),
    "pa_gemm": (c_int, [vp, vp, vp, u32, u32, f32p, u32, c_int]),
    "pa_attn_layer_prefill": (c_int, [vp, u32, vp, vp, f32p, f32p, f32p, f32p, u32, u32, u32]),
    "pa_version": (ctypes.c_char_p, []),
}

_lib = None


def load():
    """Load libpooled_attn.so and type every exported function.  Raises if the library is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libpooled_attn.so is not built (run `python -m pooled_amd.build`): %s" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


class PaError(RuntimeError):
    def __init__(self, code, msg):
        RuntimeError.__init__(self, "pooled_attn error %d: %s" % (code, msg))
        self.code = code


class DeviceBuffer:
    """A block of HBM owned through pa_malloc / pa_free."""

    def __init__(self, owner, nbytes):
        self.owner, self.nbytes = owner, int(nbytes)
        p = vp()
        owner._chk(owner.L.pa_malloc(owner.ctx, self.nbytes, ctypes.byref(p)))
        self.ptr = p.value

    def upload(self, arr, offset=0):
        a = np.ascontiguousarray(arr)
        assert offset + a.nbytes <= self.nbytes
        self.owner._chk(self.owner.L.pa_upload(self.owner.ctx, self.ptr + offset, a.ctypes.data, a.nbytes))
        return self

    def download(self, dtype, count, offset=0):
        out = np.empty(count, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        self.owner._chk(self.owner.L.pa_download(self.owner.ctx, out.ctypes.data, self.ptr + offset, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            self.owner.L.pa_free(self.owner.ctx, self.ptr)
            self.ptr = None


class PooledAttn:
    """One pa_ctx.  cfg keys: n_heads, n_kv_heads, head_dim, n_rot, rope_theta, eps, qk_norm, gate, kv_q8, verify_exact."""

    def __init__(self, cfg, max_seq, n_layers=1, max_cols=16):
        self.L = load()
        self.cfg = dict(cfg)
        flags = ((PA_FLAG_QK_NORM if cfg.get("qk_norm", True) else 0) | (PA_FLAG_GATE if cfg.get("gate", False) else 0)
                 | (PA_FLAG_KV_Q8 if cfg.get("kv_q8", False) else 0) | (PA_FLAG_VERIFY_EXACT if cfg.get("verify_exact", False) else 0))
        c = PaConfig(cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["n_rot"], cfg["rope_theta"], cfg["eps"],
                     max_seq, n_layers, max_cols, flags)
        h = vp()
        rc = self.L.pa_create(ctypes.byref(c), ctypes.byref(h))
        if rc != PA_OK:
            raise PaError(rc, (self.L.pa_last_error(None) or b"").decode())
        self.ctx = h
        self.max_seq, self.n_layers, self.max_cols = max_seq, n_layers, max_cols
        self.q_dim = cfg["n_heads"] * cfg["head_dim"]
        self.kv_dim = cfg["n_kv_heads"] * cfg["head_dim"]
        self.q_in_dim = self.q_dim * (2 if cfg.get("gate", False) else 1)
        self._bufs = []

    def _chk(self, rc):
        if rc != PA_OK:
            raise PaError(rc, (self.L.pa_last_error(self.ctx) or b"").decode())

    def close(self):
        if self.ctx:
            for w in getattr(self, "_weights", []):
                self.L.pa_weight_destroy(self.ctx, w)
            self._weights = []
            for b in self._bufs:
                b.free()
            self._bufs = []
            self.L.pa_destroy(self.ctx)
            self.ctx = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    # ---- memory ----
    def alloc(self, nbytes):
        b = DeviceBuffer(self, nbytes)
        self._bufs.append(b)
        return b

    def to_device(self, arr):
        a = np.ascontiguousarray(arr)
        return self.alloc(max(a.nbytes, 16)).upload(a)

    def copy_d2d(self, dst, src, nbytes):
        self._chk(self.L.pa_copy_d2d(self.ctx, dst.ptr, src.ptr, nbytes))

    def layer_alloc(self, layer=0):
        self._chk(self.L.pa_layer_alloc(self.ctx, layer))

    def sync(self):
        self._chk(self.L.pa_sync(self.ctx))

    # ---- cache ----
    def _kv_part(self, which):
        """(dtype, elements per kv head and row) of cache tensor `which` in the host view."""
        hd = self.cfg["head_dim"]
        if not self.cfg.get("kv_q8", False):
            return np.uint16, hd
        return (np.int8, hd) if which < 2 else (np.float32, hd // 32)

    def kv_write(self, layer, which, row0, rows):
        dt, per = self._kv_part(which)
        a = np.ascontiguousarray(rows, dtype=dt).reshape(-1, self.cfg["n_kv_heads"] * per)
        self._chk(self.L.pa_kv_write(self.ctx, layer, which, row0, a.shape[0], a.ctypes.data))

    def kv_read(self, layer, which, row0, n_rows):
        """f16 caches: f16 bits [n_rows, nKV, hd]; int8 caches: int8 values (which 0 / 1) or f32 scales
        [n_rows, nKV, hd / 32] (which 2 / 3)."""
        dt, per = self._kv_part(which)
        out = np.empty((n_rows, self.cfg["n_kv_heads"], per), dtype=dt)
        self._chk(self.L.pa_kv_read(self.ctx, layer, which, row0, n_rows, out.ctypes.data))
        return out

    # ---- launches (device buffers in, device buffers out) ----
    def glue_kv(self, layer, d_q, q_stride, d_k, k_stride, d_v, v_stride, d_qw, d_kw, base_pos, n_cols):
        self._chk(self.L.pa_glue_kv(self.ctx, layer, d_q.ptr, q_stride, d_k.ptr, k_stride, d_v.ptr, v_stride,
                                    d_qw.ptr if d_qw else None, d_kw.ptr if d_kw else None, base_pos, n_cols))

    def glue(self, d_q, q_stride, d_k, k_stride, d_qw, d_kw, base_pos, n_cols):
        self._chk(self.L.pa_glue(self.ctx, d_q.ptr, q_stride, d_k.ptr, k_stride, d_qw.ptr if d_qw else None,
                                 d_kw.ptr if d_kw else None, base_pos, n_cols))

    def kv_store(self, layer, d_k, k_stride, d_v, v_stride, base_pos, n_cols):
        self._chk(self.L.pa_kv_store(self.ctx, layer, d_k.ptr, k_stride, d_v.ptr, v_stride, base_pos, n_cols))

    def attn(self, kind, layer, d_q, q_stride, d_gate, gate_stride, base_pos, n_cols, d_out, out_stride, out_dtype=PA_OUT_F32):
        fn = self.L.pa_attn_decode if kind == "decode" else self.L.pa_attn_prefill
        qp = d_q if isinstance(d_q, (int, type(None))) else d_q.ptr
        gp = d_gate if isinstance(d_gate, (int, type(None))) else d_gate.ptr
        self._chk(fn(self.ctx, layer, qp, q_stride, gp, gate_stride, base_pos, n_cols, d_out.ptr, out_stride, out_dtype))

    def attn_decode_step(self, layer, d_q_in, d_k, d_v, d_qw, d_kw, pos, d_out, out_dtype=PA_OUT_F32, noalloc=False):
        fn = self.L.pa_attn_decode_step_noalloc if noalloc else self.L.pa_attn_decode_step
        self._chk(fn(self.ctx, layer, d_q_in.ptr, d_k.ptr, d_v.ptr, d_qw.ptr if d_qw else None,
                                             d_kw.ptr if d_kw else None, pos, d_out.ptr, out_dtype))

    def q_buffer_ptr(self):
        return self.L.pa_q_buffer(self.ctx)

    def gate_buffer_ptr(self):
        return self.L.pa_gate_buffer(self.ctx)

    def read_q_buffer(self, n_cols):
        out = np.empty((n_cols, self.cfg["n_heads"], self.cfg["head_dim"]), dtype=np.float32)
        self._chk(self.L.pa_download(self.ctx, out.ctypes.data, self.q_buffer_ptr(), out.nbytes))
        return out

    def read_gate_buffer(self, n_cols):
        out = np.empty((n_cols, self.cfg["n_heads"], self.cfg["head_dim"]), dtype=np.float32)
        self._chk(self.L.pa_download(self.ctx, out.ctypes.data, self.gate_buffer_ptr(), out.nbytes))
        return out

    def plan(self, kind, base_pos, n_cols):
        pl = PaPlan()
        self._chk(self.L.pa_plan_query(self.ctx, 0 if kind == "decode" else 1, base_pos, n_cols, ctypes.byref(pl)))
        return {n: getattr(pl, n) for n, _ in PaPlan._fields_}

    def set_decode_splits(self, n):
        self._chk(self.L.pa_set_decode_splits(self.ctx, n))

    def set_prefill_tile(self, mode):
        """0: the table picks the kernel of a prefill chunk, 1: always the matrix-core kernel, 2: never."""
        self._chk(self.L.pa_set_prefill_tile(self.ctx, mode))

    def set_weight_cache(self, max_bytes):
        """Budget of the f16 weight copies that large-chunk gemm calls keep with their weight handles (0: keep none)."""
        self._chk(self.L.pa_set_weight_cache(self.ctx, max_bytes))

    # ---- timing ----
    def timer_start(self):
        self._chk(self.L.pa_timer_start(self.ctx))

    def timer_stop(self):
        ms = ctypes.c_float()
        self._chk(self.L.pa_timer_stop(self.ctx, ctypes.byref(ms)))
        return ms.value

    def profile_enable(self, on=True):
        self._chk(self.L.pa_profile_enable(self.ctx, 1 if on else 0))

    def profile_read(self):
        ms, n = ctypes.c_float(), u32()
        self._chk(self.L.pa_profile_read(self.ctx, ctypes.byref(ms), ctypes.byref(n)))
        return ms.value, n.value

    def profile_read_each(self, cap=4096):
        """Durations (ms) of the main-kernel launches timed since the last read, in launch order."""
        buf, n = (ctypes.c_float * cap)(), u32()
        self._chk(self.L.pa_profile_read_each(self.ctx, buf, cap, ctypes.byref(n)))
        return [buf[i] for i in range(min(n.value, cap))]

    # ---- checkpoint slots ----
    def slot_save(self, slot, pos):
        self._chk(self.L.pa_slot_save(self.ctx, slot, pos))

    def slot_load(self, slot):
        pos = u32()
        self._chk(self.L.pa_slot_load(self.ctx, slot, ctypes.byref(pos)))
        return pos.value

    def slot_drop(self, slot):
        self._chk(self.L.pa_slot_drop(self.ctx, slot))

    def slot_pos(self, slot):
        pos = u32()
        self._chk(self.L.pa_slot_pos(self.ctx, slot, ctypes.byref(pos)))
        return pos.value

    def slot_create(self, slot, pos):
        self._chk(self.L.pa_slot_create(self.ctx, slot, pos))

    def slot_export(self, slot, layer, which):
        """One part, position-major [pos, nKV * row]: f16 bits, or int8 values / f32 scales on an int8 cache."""
        dt, per = self._kv_part(which)
        out = np.empty((self.slot_pos(slot), self.cfg["n_kv_heads"] * per), dtype=dt)
        self._chk(self.L.pa_slot_export(self.ctx, slot, layer, which, out.ctypes.data))
        return out

    def slot_import(self, slot, layer, which, part):
        part = np.ascontiguousarray(part, dtype=self._kv_part(which)[0])
        self._chk(self.L.pa_slot_import(self.ctx, slot, layer, which, part.ctypes.data))

    # ---- projections (one-token passes) ----
    def weight(self, kind, w, scales=None):
        """Upload a weight matrix: kind PA_W_F32 (w f32 [d_out, d_in]), PA_W_Q8_0 (w int8 [d_out, d_in]) or PA_W_Q4_0
        (w uint8 [d_out, d_in / 2]); scales: f16 bits (uint16) [d_out, d_in / 32].  Returns an opaque handle."""
        w = np.ascontiguousarray(w)
        d_out = w.shape[0]
        d_in = w.shape[1] * (2 if kind == PA_W_Q4_0 else 1)
        sc = None if scales is None else np.ascontiguousarray(scales, dtype=np.uint16)
        h = vp()
        self._chk(self.L.pa_weight_create(self.ctx, kind, d_out, d_in, w.ctypes.data, sc.ctypes.data if sc is not None else None, ctypes.byref(h)))
        if not hasattr(self, "_weights"):
            self._weights = []
        self._weights.append(h)
        return h

    def gemv(self, w, d_x, d_y, acc=False):
        self._chk(self.L.pa_gemv(self.ctx, w, d_x.ptr, d_y.ptr, int(bool(acc))))

    def gemv_norm(self, w, d_x_raw, d_norm_w, d_y, d_xn_out=None):
        self._chk(self.L.pa_gemv_norm(self.ctx, w, d_x_raw.ptr, d_norm_w.ptr, d_xn_out.ptr if d_xn_out else None, d_y.ptr))

    def attn_layer_decode(self, layer, w_qkv, w_o, d_attn_norm_w, d_qw, d_kw, d_x, pos):
        self._chk(self.L.pa_attn_layer_decode(self.ctx, layer, w_qkv, w_o, d_attn_norm_w.ptr, d_qw.ptr if d_qw else None,
                                              d_kw.ptr if d_kw else None, d_x.ptr, pos))

    def rmsnorm_f16(self, d_x, x_stride, d_norm_w, dim, n_cols, d_xn, xn_stride):
        self._chk(self.L.pa_rmsnorm_f16(self.ctx, d_x.ptr, x_stride, d_norm_w.ptr, dim, n_cols, d_xn.ptr, xn_stride))

    def gemm(self, w, d_x16, x_stride, n_cols, d_y, y_stride, acc=False):
        self._chk(self.L.pa_gemm(self.ctx, w, d_x16.ptr, x_stride, n_cols, d_y.ptr, y_stride, int(bool(acc))))

    def attn_layer_prefill(self, layer, w_qkv, w_o, d_attn_norm_w, d_qw, d_kw, d_x, x_stride, base_pos, n_cols):
        self._chk(self.L.pa_attn_layer_prefill(self.ctx, layer, w_qkv, w_o, d_attn_norm_w.ptr, d_qw.ptr if d_qw else None,
                                               d_kw.ptr if d_kw else None, d_x.ptr, x_stride, base_pos, n_cols))

    # ---- numpy convenience used by tests / smoke: whole passes from host arrays ----
    def run_glue_kv(self, layer, q_in, k_in, v_in, qw, kw, base_pos):
        n = q_in.shape[0]
        dq, dk, dv = self.to_device(q_in.astype(np.float32)), self.to_device(k_in.astype(np.float32)), self.to_device(v_in.astype(np.float32))
        dqw, dkw = self.to_device(qw.astype(np.float32)), self.to_device(kw.astype(np.float32))
        self.glue_kv(layer, dq, q_in.shape[1], dk, k_in.shape[1], dv, v_in.shape[1], dqw, dkw, base_pos, n)
        self.sync()
        for b in (dq, dk, dv, dqw, dkw):
            b.free(); self._bufs.remove(b)

    def run_decode_step(self, layer, q_in, k_in, v_in, qw, kw, pos, out_dtype=PA_OUT_F32):
        """One decode token through the fused entry point: q_in [qcol], k_in / v_in [nKV*hd] f32 -> out [nH, hd]."""
        bufs = [self.to_device(np.ascontiguousarray(a, dtype=np.float32)) for a in (q_in, k_in, v_in, qw, kw)]
        esz = 4 if out_dtype == PA_OUT_F32 else 2
        dout = self.alloc(self.q_dim * esz)
        self.attn_decode_step(layer, bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], pos, dout, out_dtype)
        self.sync()
        out = dout.download(np.float32 if out_dtype == PA_OUT_F32 else np.float16, self.q_dim)
        for b in bufs + [dout]:
            b.free(); self._bufs.remove(b)
        return out.reshape(self.cfg["n_heads"], self.cfg["head_dim"])

    def run_attn_gather(self, layer, q, lists, gate=None, out_dtype=PA_OUT_F32):
        """q [n, nH, hd]; lists: n sequences of cache row indices (ascending) -> out [n, nH, hd]."""
        n = q.shape[0]
        max_rows = max(len(l) for l in lists)
        stride = max_rows + 1
        sel = np.zeros((n, stride), np.uint32)
        for c, l in enumerate(lists):
            sel[c, 0] = len(l); sel[c, 1:1 + len(l)] = np.asarray(l, np.uint32)
        dq = self.to_device(q.reshape(n, -1).astype(np.float32))
        dg = self.to_device(gate.reshape(n, -1).astype(np.float32)) if gate is not None else None
        dsel = self.to_device(sel)
        esz = 4 if out_dtype == PA_OUT_F32 else 2
        dout = self.alloc(n * self.q_dim * esz)
        self._chk(self.L.pa_attn_decode_gather(self.ctx, layer, dq.ptr, self.q_dim, dg.ptr if dg else None, self.q_dim if dg else 0,
                                               dsel.ptr, stride, max_rows, n, dout.ptr, self.q_dim, out_dtype))
        self.sync()
        out = dout.download(np.float32 if out_dtype == PA_OUT_F32 else np.float16, n * self.q_dim)
        for b in (dq, dg, dsel, dout):
            if b is not None:
                b.free(); self._bufs.remove(b)
        return out.reshape(n, self.cfg["n_heads"], self.cfg["head_dim"])

    def run_attn(self, kind, layer, q, base_pos, gate=None, out_dtype=PA_OUT_F32):
        """q [n, nH, hd] f32 (None: the context's q buffer, n from gate or 1) -> out [n, nH, hd]."""
        n = q.shape[0]
        dq = self.to_device(q.reshape(n, -1).astype(np.float32))
        dg = self.to_device(gate.reshape(n, -1).astype(np.float32)) if gate is not None else None
        esz = 4 if out_dtype == PA_OUT_F32 else 2
        dout = self.alloc(n * self.q_dim * esz)
        self.attn(kind, layer, dq, self.q_dim, dg, self.q_dim if dg else 0, base_pos, n, dout, self.q_dim, out_dtype)
        self.sync()
        out = dout.download(np.float32 if out_dtype == PA_OUT_F32 else np.float16, n * self.q_dim)
        for b in (dq, dg, dout):
            if b is not None:
                b.free(); self._bufs.remove(b)
        return out.reshape(n, self.cfg["n_heads"], self.cfg["head_dim"])
