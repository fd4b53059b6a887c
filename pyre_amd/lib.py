"""ctypes binding of libpyre_hip.so (include/pyre_hip.h) plus thin host-side mirrors of the reference's types:
QMat (src/model/gguf_q.rs:201-247).  There is no CPU fallback: a missing library or a failing call raises."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("PYRE_LIB") or os.path.join(_HERE, "csrc", "libpyre_hip.so")      # PYRE_LIB: another build of the library (diagnostics variants)

F32, F16, Q8_0, Q4_K, IQ2_XS, IQ3_S, BF16 = 0, 1, 8, 12, 17, 21, 30
Q4_0, Q5_0, Q6_K, IQ2_XXS, IQ3_XXS, IQ4_NL, IQ2_S, IQ4_XS, Q3_K, Q2_0, Q5_K, IQ1_M = 2, 6, 14, 16, 18, 20, 22, 23, 11, 42, 13, 29      # re-coded at load (scale x small integer)

_lib = None


class PyreError(RuntimeError):
    pass


def _declare(L):
    vp, sz, u32, u64, i32, f32 = C.c_void_p, C.c_size_t, C.c_uint32, C.c_uint64, C.c_int, C.c_float
    sig = {
        "pyre_ctx_create": (i32, [i32, C.POINTER(vp)]),
        "pyre_ctx_destroy": (None, [vp]),
        "pyre_last_error": (C.c_char_p, [vp]),
        "pyre_ctx_sync": (i32, [vp]),
        "pyre_ctx_stream": (vp, [vp]),
        "pyre_prof_enable": (i32, [vp, i32]),
        "pyre_prof_reset": (i32, [vp]),
        "pyre_prof_report": (C.c_char_p, [vp]),
        "pyre_dev_alloc": (i32, [vp, sz, C.POINTER(vp)]),
        "pyre_dev_free": (i32, [vp, vp]),
        "pyre_dev_upload": (i32, [vp, vp, vp, sz]),
        "pyre_dev_download": (i32, [vp, vp, vp, sz]),
        "pyre_qmat_create": (i32, [vp, u32, sz, sz, vp, sz, C.POINTER(vp)]),
        "pyre_qmat_create_dev": (i32, [vp, u32, sz, sz, vp, sz, C.POINTER(vp)]),
        "pyre_qmat_destroy": (None, [vp]),
        "pyre_qmat_rows": (sz, [vp]),
        "pyre_qmat_cols": (sz, [vp]),
        "pyre_qmat_gguf_bytes": (sz, [vp]),
        "pyre_qmat_device_bytes": (sz, [vp]),
        "pyre_qmat_dequant": (i32, [vp, vp, vp]),
        "pyre_qmat_dequant_dev": (i32, [vp, vp, vp]),
        "pyre_qmat_row": (i32, [vp, vp, sz, vp]),
        "pyre_qmatmul": (i32, [vp, vp, vp, i32, vp]),
        "pyre_qmatmul_dev": (i32, [vp, vp, vp, i32, vp]),
        "pyre_qmatmul_f32": (i32, [vp, vp, vp, i32, vp]),
        "pyre_qmatmul_f32_dev": (i32, [vp, vp, vp, i32, vp]),
        "pyre_qmatmul_static_dev": (i32, [vp, vp, vp, i32, vp]),
        "pyre_qmat_layout_bytes": (sz, [vp, i32]),
        "pyre_gguf_open": (i32, [C.c_char_p, vp, C.c_char_p, C.c_size_t]),
        "pyre_gguf_close": (None, [vp]),
        "pyre_gguf_n_shards": (C.c_size_t, [vp]),
        "pyre_gguf_n_tensors": (C.c_size_t, [vp]),
        "pyre_gguf_tensor_name": (C.c_char_p, [vp, C.c_size_t]),
        "pyre_gguf_has": (i32, [vp, C.c_char_p]),
        "pyre_gguf_tensor": (i32, [vp, C.c_char_p, vp, vp, vp, C.c_char_p, C.c_size_t]),
        "pyre_gguf_meta_u64": (i32, [vp, C.c_char_p, vp]),
        "pyre_gguf_meta_f64": (i32, [vp, C.c_char_p, vp]),
        "pyre_gguf_meta_str": (i32, [vp, C.c_char_p, C.c_char_p, C.c_size_t]),
        "pyre_gguf_meta_arr_u64": (C.c_long, [vp, C.c_char_p, vp, C.c_size_t]),
        "pyre_session_create": (i32, [vp, vp, i32, i32, sz, C.POINTER(vp)]),
        "pyre_session_destroy": (None, [vp]),
        "pyre_session_state": (vp, [vp]),
        "pyre_session_prefill": (i32, [vp, vp, vp, i32, vp, C.POINTER(i32), C.POINTER(i32)]),
        "pyre_session_generate_greedy": (i32, [vp, vp, vp, i32, vp, i32, vp, C.POINTER(i32)]),
        "pyre_session_stats": (i32, [vp, C.POINTER(i32), C.POINTER(sz), C.POINTER(i32)]),
        "pyre_session_snapshot_len": (i32, [vp, i32]),
        "pyre_model_load_gguf": (i32, [vp, C.c_char_p, i32, i32, i32, vp]),
        "pyre_state_capacity": (i32, [vp]),
        "pyre_model_max_window": (i32, [vp]),
        "pyre_state_snapshot": (i32, [vp, vp, vp]),
        "pyre_state_restore": (i32, [vp, vp, vp]),
        "pyre_snap_destroy": (None, [vp]),
        "pyre_snap_bytes": (C.c_size_t, [vp]),
        "pyre_snap_len": (i32, [vp]),
        "pyre_synth_blocks": (i32, [vp, u32, sz, u64, f32, f32, vp]),
        "pyre_moe_create": (i32, [vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, C.POINTER(vp)]),
        "pyre_moe_destroy": (None, [vp]),
        "pyre_moe_ffn": (i32, [vp, vp, vp, i32, vp, vp, vp]),
        "pyre_moe_ffn_dev": (i32, [vp, vp, vp, i32, vp]),
        "pyre_gdn_create": (i32, [vp, i32, i32, i32, i32, i32, f32, vp, vp, vp, vp, C.POINTER(vp)]),
        "pyre_gdn_destroy": (None, [vp]),
        "pyre_gdn_set_state": (i32, [vp, vp, vp, vp]),
        "pyre_gdn_get_state": (i32, [vp, vp, vp, vp]),
        "pyre_gdn_step": (i32, [vp, vp, vp, i32, vp]),
        "pyre_gdn_prefill_chunked": (i32, [vp, vp, vp, i32, i32, vp]),
        "pyre_attn_create": (i32, [vp, i32, i32, i32, i32, f32, f32, vp, vp, i32, i32, i32, C.POINTER(vp)]),
        "pyre_attn_destroy": (None, [vp]),
        "pyre_attn_len": (i32, [vp]),
        "pyre_attn_truncate": (i32, [vp, vp, i32]),
        "pyre_attn_decode_kv4": (i32, [vp, vp, vp, i32, vp]),
        "pyre_attn_load_cache": (i32, [vp, vp, vp, vp, i32]),
        "pyre_attn_read_cache": (i32, [vp, vp, vp, vp]),
        "pyre_attn_set_indexer": (i32, [vp, vp, i32, i32, i32, i32, vp, vp]),
        "pyre_attn_set_context": (i32, [vp, vp, i32, i32]),
        "pyre_attn_load_index": (i32, [vp, vp, vp]),
        "pyre_attn_read_index": (i32, [vp, vp, vp, vp]),
        "pyre_attn_read_selection": (i32, [vp, vp, i32, vp, i32, vp]),
        "pyre_model_create": (i32, [vp, vp, vp, vp, C.POINTER(vp)]),
        "pyre_model_destroy": (None, [vp]),
        "pyre_model_weight_bytes_per_token": (sz, [vp]),
        "pyre_model_prompt_blocks": (sz, [vp]),
        "pyre_state_create": (i32, [vp, vp, i32, C.POINTER(vp)]),
        "pyre_state_destroy": (None, [vp]),
        "pyre_state_reset": (i32, [vp, vp]),
        "pyre_state_len": (i32, [vp]),
        "pyre_state_read_gdn": (i32, [vp, vp, i32, vp, vp]),
        "pyre_state_read_kv": (i32, [vp, vp, i32, vp, vp]),
        "pyre_state_read_ple": (i32, [vp, vp, i32, vp]),
        "pyre_forward": (i32, [vp, vp, vp, vp, i32, vp]),
        "pyre_forward_multi": (i32, [vp, vp, vp, vp, i32, vp]),
        "pyre_spec_keep": (i32, [vp, vp, vp, i32, i32]),
        "pyre_generate_greedy": (i32, [vp, vp, vp, vp, i32, vp, i32, vp, C.POINTER(i32)]),
        "pyre_ngram_draft": (i32, [vp, C.c_size_t, i32, i32, i32, vp]),
        "pyre_argmax_rows": (i32, [vp, vp, i32, i32, vp]),
        "pyre_generate_greedy_ngram": (i32, [vp, vp, vp, vp, C.c_size_t, vp, i32, vp, i32, i32, i32, C.POINTER(i32), C.POINTER(i32), C.POINTER(i32)]),
        "pyre_decode_greedy_dev": (i32, [vp, vp, vp, u32, i32, vp]),
        "pyre_mtp_create": (i32, [vp, vp, vp, vp, vp, C.POINTER(vp)]),
        "pyre_mtp_destroy": (None, [vp]),
        "pyre_state_attach_mtp": (i32, [vp, vp, vp]),
        "pyre_mtp_draft": (i32, [vp, vp, vp, u32, i32, f32, vp, vp, C.POINTER(i32)]),
        "pyre_mtp_read_kv": (i32, [vp, vp, C.POINTER(i32), C.POINTER(i32), vp, vp]),
        "pyre_generate_greedy_mtp": (i32, [vp, vp, vp, vp, vp, i32, vp, i32, f32, C.POINTER(i32), C.POINTER(i32), C.POINTER(i32)]),
        "pyre_generate_greedy_mtp_forced": (i32, [vp, vp, vp, vp, vp, i32, vp, i32, vp, C.POINTER(i32), C.POINTER(i32), C.POINTER(i32)]),
        "pyre_adapt_plan": (i32, [i32, C.c_double, vp, C.c_double, C.c_double]),
        "pyre_spec_set_adapt": (None, [vp, i32]),
        "pyre_st_open": (i32, [C.c_char_p, C.POINTER(vp), C.c_char_p, C.c_size_t]),
        "pyre_st_close": (None, [vp]),
        "pyre_st_n_tensors": (C.c_size_t, [vp]),
        "pyre_st_tensor_name": (C.c_char_p, [vp, C.c_size_t]),
        "pyre_st_tensor": (i32, [vp, C.c_char_p, C.POINTER(vp), C.POINTER(u32), vp, C.c_char_p, C.c_size_t]),
        "pyre_mtp_load_safetensors": (i32, [vp, vp, C.c_char_p, i32, i32, vp, i32, vp, C.POINTER(vp)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    return sig


def exported_symbols():
    """Names include/pyre_hip.h declares (parsed from the header itself)."""
    import re
    hdr = open(os.path.join(os.path.dirname(_HERE), "include", "pyre_hip.h")).read()
    return sorted(set(re.findall(r"\b(pyre_[a-z0-9_]+)\s*\(", hdr)))


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise PyreError("libpyre_hip.so is not built: run `python -c 'import __graft_entry__ as g; g.build()'` (%s)" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        _declare(L)
        _lib = L
    return _lib


def ngram_draft(history, k, min_n, max_n):
    """spec::ngram_draft through the library (host only, needs no GPU)."""
    h = np.ascontiguousarray(history, dtype=np.uint32); out = np.empty(max(k, 1), dtype=np.uint32)
    n = load().pyre_ngram_draft(h.ctypes.data_as(C.c_void_p), h.size, k, min_n, max_n, out.ctypes.data_as(C.c_void_p))
    return out[:n].copy()


def adapt_plan(n, ts, tv, p, td):
    """spec::adapt_plan through the library (host only, needs no GPU); tv: ten verify times, 0 = unmeasured."""
    t = np.ascontiguousarray(tv, dtype=np.float64); assert t.size == 10
    return int(load().pyre_adapt_plan(n, ts, t.ctypes.data_as(C.c_void_p), p, td))


class Safetensors:
    """The drafter checkpoint's container (St of src/model/mtp.rs) through the library (host only, needs no GPU)."""

    def __init__(self, path):
        self.L = load(); h = C.c_void_p(); err = C.create_string_buffer(512)
        rc = self.L.pyre_st_open(os.fsencode(path), C.byref(h), err, 512)
        if rc != 0:
            raise PyreError("pyre_st_open (%d): %s" % (rc, err.value.decode()))
        self.h = h; self.rc = rc

    def names(self):
        return [self.L.pyre_st_tensor_name(self.h, i).decode() for i in range(self.L.pyre_st_n_tensors(self.h))]

    def tensor(self, name):
        """(shape, raw bf16 bits as a uint16 array)"""
        d = C.c_void_p(); nd = C.c_uint32(); dims = (C.c_uint64 * 8)(); err = C.create_string_buffer(512)
        rc = self.L.pyre_st_tensor(self.h, name.encode(), C.byref(d), C.byref(nd), dims, err, 512)
        if rc != 0:
            raise PyreError("pyre_st_tensor (%d): %s" % (rc, err.value.decode()))
        shape = [int(dims[i]) for i in range(nd.value)]; n = int(np.prod(shape)) if shape else 1
        return shape, np.ctypeslib.as_array(C.cast(d, C.POINTER(C.c_uint16)), shape=(n,)).copy()

    def close(self):
        if self.h:
            self.L.pyre_st_close(self.h); self.h = None


def _ptr(a):
    if a is None:
        return None
    if isinstance(a, np.ndarray):
        return a.ctypes.data_as(C.c_void_p)
    if isinstance(a, int):
        return C.c_void_p(a)
    if hasattr(a, "data_ptr"):      # torch tensor on the context's device
        return C.c_void_p(a.data_ptr())
    raise TypeError(type(a))


class Context:
    def __init__(self, device=0):
        self.L = load()
        h = C.c_void_p()
        rc = self.L.pyre_ctx_create(device, C.byref(h))
        if rc != 0:
            raise PyreError("pyre_ctx_create: %s" % self.L.pyre_last_error(None).decode())
        self.h = h

    def check(self, rc, what=""):
        if rc != 0:
            raise PyreError("%s failed (%d): %s" % (what, rc, self.L.pyre_last_error(self.h).decode()))

    def sync(self):
        self.check(self.L.pyre_ctx_sync(self.h), "sync")

    def set_spec_adapt(self, on):
        """Adaptive draft length of the drafted greedy loops (spec::adapt_on): 1 / 0, or -1 = PYRE_SPEC_ADAPT."""
        self.L.pyre_spec_set_adapt(self.h, int(on))

    @property
    def stream(self):
        return self.L.pyre_ctx_stream(self.h)

    def alloc(self, nbytes):
        p = C.c_void_p()
        self.check(self.L.pyre_dev_alloc(self.h, nbytes, C.byref(p)), "dev_alloc")
        return p.value

    def free(self, p):
        self.check(self.L.pyre_dev_free(self.h, C.c_void_p(p)), "dev_free")

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        p = self.alloc(arr.nbytes)
        self.check(self.L.pyre_dev_upload(self.h, C.c_void_p(p), _ptr(arr), arr.nbytes), "upload")
        return p

    def download(self, p, shape, dtype=np.float32):
        out = np.empty(shape, dtype=dtype)
        self.check(self.L.pyre_dev_download(self.h, _ptr(out), C.c_void_p(p), out.nbytes), "download")
        return out

    def synth_blocks(self, ty, n_blocks, seed, d_lo=1e-3, d_hi=2e-2, dev_out=None):
        self.check(self.L.pyre_synth_blocks(self.h, ty, n_blocks, seed, d_lo, d_hi, C.c_void_p(dev_out)), "synth_blocks")

    def prof_enable(self, on=True):
        self.check(self.L.pyre_prof_enable(self.h, 1 if on else 0), "prof_enable")

    def prof_reset(self):
        self.check(self.L.pyre_prof_reset(self.h), "prof_reset")

    def prof_report(self):
        """{kernel class: (launches, total_ms, algorithmic_bytes)}"""
        out = {}
        for line in self.L.pyre_prof_report(self.h).decode().splitlines():
            name, n, ms, by = line.split()
            out[name] = (int(n), float(ms), float(by))
        return out

    def close(self):
        if getattr(self, "h", None):
            self.L.pyre_ctx_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class QMat:
    """Quantized row-major matrix on the device: `rows` rows of `cols` elements of ggml type `ty`."""

    def __init__(self, ctx, ty, rows, cols, blocks=None, dev_blocks=None, nbytes=None):
        self.ctx = ctx
        self.ty, self.rows, self.cols = ty, rows, cols
        h = C.c_void_p()
        if blocks is not None:
            blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
            rc = ctx.L.pyre_qmat_create(ctx.h, ty, rows, cols, _ptr(blocks), blocks.nbytes, C.byref(h))
        else:
            rc = ctx.L.pyre_qmat_create_dev(ctx.h, ty, rows, cols, C.c_void_p(dev_blocks), nbytes, C.byref(h))
        ctx.check(rc, "qmat_create")
        self.h = h

    @property
    def gguf_bytes(self):
        return self.ctx.L.pyre_qmat_gguf_bytes(self.h)

    @property
    def dev_bytes(self):
        return self.ctx.L.pyre_qmat_device_bytes(self.h)

    def layout_bytes(self, layout):
        """Device bytes of one layout: 0 / False = the lane-per-row planes, 1 / True = the matrix-core layout (IQ3_S only),
        2 = IQ3_S at the file's bits per weight (what a single-token matmul streams)."""
        return self.ctx.L.pyre_qmat_layout_bytes(self.h, int(layout))

    def to_f32(self):
        out = np.empty((self.rows, self.cols), dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_qmat_dequant(self.ctx.h, self.h, _ptr(out)), "qmat_dequant")
        return out

    def row(self, r):
        out = np.empty(self.cols, dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_qmat_row(self.ctx.h, self.h, r, _ptr(out)), "qmat_row")
        return out

    def matmul(self, x, t=None):
        """y[ti, r] = sum_c W[r, c] x[ti, c]; x is a host array [t, cols]."""
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.cols)
        t = x.shape[0] if t is None else t
        y = np.empty((t, self.rows), dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_qmatmul(self.ctx.h, self.h, _ptr(x), t, _ptr(y)), "qmatmul")
        return y

    def matmul_f32(self, x):
        """matmul on the f32 multiply-add GEMV the model's expert matrices use (IQ3_S: matmul itself takes the native-format integer-dot kernel for one token and the matrix cores for a window)."""
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.cols)
        y = np.empty((x.shape[0], self.rows), dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_qmatmul_f32(self.ctx.h, self.h, _ptr(x), x.shape[0], _ptr(y)), "qmatmul_f32")
        return y

    def matmul_static_dev(self, x_dev, t, y_dev):
        """pyre_qmatmul_static_dev: device pointers in and out, nothing allocated by the call."""
        self.ctx.check(self.ctx.L.pyre_qmatmul_static_dev(self.ctx.h, self.h, _ptr(x_dev), t, _ptr(y_dev)), "qmatmul_static_dev")

    def matmul_dev(self, x_dev, t, y_dev):
        self.ctx.check(self.ctx.L.pyre_qmatmul_dev(self.ctx.h, self.h, _ptr(x_dev), t, _ptr(y_dev)), "qmatmul_dev")

    def matmul_f32_dev(self, x_dev, t, y_dev):
        self.ctx.check(self.ctx.L.pyre_qmatmul_f32_dev(self.ctx.h, self.h, _ptr(x_dev), t, _ptr(y_dev)), "qmatmul_f32_dev")

    def close(self):
        if getattr(self, "h", None) and getattr(self.ctx, "h", None):
            self.ctx.L.pyre_qmat_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Moe:
    """MoE FFN block over borrowed QMats (ffn / routed of the reference, qwen4exp_gguf.rs:1675-1795)."""

    def __init__(self, ctx, top_k, router, gate_e, up_e, down_e, sh_gate_inp, sh_gate, sh_up, sh_down):
        self.ctx = ctx
        self._keep = (router, gate_e, up_e, down_e, sh_gate, sh_up, sh_down)
        self.d, self.top_k = router.cols, top_k
        sgi = np.ascontiguousarray(sh_gate_inp, dtype=np.float32)
        h = C.c_void_p()
        ctx.check(ctx.L.pyre_moe_create(ctx.h, top_k, router.h, gate_e.h, up_e.h, down_e.h, _ptr(sgi), sh_gate.h, sh_up.h, sh_down.h, C.byref(h)), "moe_create")
        self.h = h

    def ffn(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, self.d)
        t = x.shape[0]
        y = np.empty((t, self.d), dtype=np.float32)
        idx = np.empty((t, self.top_k), dtype=np.int32)
        w = np.empty((t, self.top_k), dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_moe_ffn(self.ctx.h, self.h, _ptr(x), t, _ptr(y), _ptr(idx), _ptr(w)), "moe_ffn")
        return y, idx, w

    def ffn_dev(self, x_dev, t, y_dev):
        self.ctx.check(self.ctx.L.pyre_moe_ffn_dev(self.ctx.h, self.h, _ptr(x_dev), t, _ptr(y_dev)), "moe_ffn_dev")

    def close(self):
        if getattr(self, "h", None) and getattr(self.ctx, "h", None):
            self.ctx.L.pyre_moe_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Gdn:
    """Gated DeltaNet layer core with its resident recurrent state (linear_core, qwen4exp_gguf.rs:1624-1673)."""

    def __init__(self, ctx, nk, nv, dk, dv, conv_k, eps, a, dt, conv_w, norm_w):
        self.ctx = ctx
        self.nk, self.nv, self.dk, self.dv, self.conv_k = nk, nv, dk, dv, conv_k
        self.ch = 2 * nk * dk + nv * dv
        self.pw = self.ch + nv * dv + 2 * nv
        f = lambda v: np.ascontiguousarray(v, dtype=np.float32)
        a, dt, conv_w, norm_w = f(a), f(dt), f(conv_w), f(norm_w)
        h = C.c_void_p()
        ctx.check(ctx.L.pyre_gdn_create(ctx.h, nk, nv, dk, dv, conv_k, eps, _ptr(a), _ptr(dt), _ptr(conv_w), _ptr(norm_w), C.byref(h)), "gdn_create")
        self.h = h

    def set_state(self, conv=None, ssm=None):
        f = lambda v: None if v is None else np.ascontiguousarray(v, dtype=np.float32)
        conv, ssm = f(conv), f(ssm)
        self.ctx.check(self.ctx.L.pyre_gdn_set_state(self.ctx.h, self.h, _ptr(conv), _ptr(ssm)), "gdn_set_state")

    def get_state(self):
        conv = np.empty(((self.conv_k - 1), self.ch), dtype=np.float32)
        ssm = np.empty((self.nv, self.dk, self.dv), dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_gdn_get_state(self.ctx.h, self.h, _ptr(conv), _ptr(ssm)), "gdn_get_state")
        return conv, ssm

    def step(self, qkv, z, beta, alpha):
        proj = np.ascontiguousarray(np.concatenate([qkv, z, beta, alpha], axis=1), dtype=np.float32)
        t = proj.shape[0]
        assert proj.shape[1] == self.pw
        out = np.empty((t, self.nv * self.dv), dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_gdn_step(self.ctx.h, self.h, _ptr(proj), t, _ptr(out)), "gdn_step")
        return out

    def prefill_chunked(self, qkv, z, beta, alpha, chunk=64):
        proj = np.ascontiguousarray(np.concatenate([qkv, z, beta, alpha], axis=1), dtype=np.float32)
        t = proj.shape[0]
        out = np.empty((t, self.nv * self.dv), dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_gdn_prefill_chunked(self.ctx.h, self.h, _ptr(proj), t, chunk, _ptr(out)), "gdn_prefill_chunked")
        return out

    def close(self):
        if getattr(self, "h", None) and getattr(self.ctx, "h", None):
            self.ctx.L.pyre_gdn_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Attn:
    """Gated attention layer core over its own KV cache (attn_core dense branch, qwen4exp_gguf.rs:1558-1615)."""

    def __init__(self, ctx, nh, nkv, hd, n_rot, rope_base, eps, qn, kn, kv_bits, kv_recent, max_ctx):
        self.ctx = ctx
        self.nh, self.nkv, self.hd = nh, nkv, hd
        qn = np.ascontiguousarray(qn, dtype=np.float32); kn = np.ascontiguousarray(kn, dtype=np.float32)
        h = C.c_void_p()
        ctx.check(ctx.L.pyre_attn_create(ctx.h, nh, nkv, hd, n_rot, rope_base, eps, _ptr(qn), _ptr(kn), kv_bits, kv_recent, max_ctx, C.byref(h)), "attn_create")
        self.h = h

    def __len__(self):
        return self.ctx.L.pyre_attn_len(self.h)

    def truncate(self, n):
        self.ctx.check(self.ctx.L.pyre_attn_truncate(self.ctx.h, self.h, n), "attn_truncate")

    def load_cache(self, k, v):
        k = np.ascontiguousarray(k, dtype=np.float32); v = np.ascontiguousarray(v, dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_attn_load_cache(self.ctx.h, self.h, _ptr(k), _ptr(v), k.shape[0]), "attn_load_cache")

    def read_cache(self):
        n = len(self)
        k = np.empty((n, self.nkv * self.hd), dtype=np.float32); v = np.empty_like(k)
        self.ctx.check(self.ctx.L.pyre_attn_read_cache(self.ctx.h, self.h, _ptr(k), _ptr(v)), "attn_read_cache")
        return k, v

    def set_indexer(self, idx_nh, idx_hd, idx_ratio, idx_budget, iqn, ikn):
        """QSA sparse indexer (qwen4exp_gguf.rs:1565-1599); decode() then also takes the raw index projections."""
        iqn = np.ascontiguousarray(iqn, dtype=np.float32); ikn = np.ascontiguousarray(ikn, dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_attn_set_indexer(self.ctx.h, self.h, idx_nh, idx_hd, idx_ratio, idx_budget, _ptr(iqn), _ptr(ikn)), "attn_set_indexer")
        self.idx = (idx_nh, idx_hd, idx_ratio, idx_budget)

    def set_context(self, ctx_train, ctx_tokens):
        self.ctx.check(self.ctx.L.pyre_attn_set_context(self.ctx.h, self.h, ctx_train, ctx_tokens), "attn_set_context")

    def load_index(self, ik):
        ik = np.ascontiguousarray(ik, dtype=np.float32); assert ik.shape[0] == len(self)
        self.ctx.check(self.ctx.L.pyre_attn_load_index(self.ctx.h, self.h, _ptr(ik)), "attn_load_index")

    def read_index(self):
        nh, hd, ratio, _ = self.idx; n = len(self)
        ik = np.empty((n, hd), dtype=np.float32); ib = np.empty((n // ratio, hd), dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_attn_read_index(self.ctx.h, self.h, _ptr(ik), _ptr(ib)), "attn_read_index")
        return ik, ib

    def selection(self, ti):
        """Positions the last decode call attended to for its token ti (None: every visible position)."""
        _, _, ratio, budget = self.idx
        pos = np.empty(budget + 2 * ratio + 4, dtype=np.int32); cnt = C.c_int32()
        self.ctx.check(self.ctx.L.pyre_attn_read_selection(self.ctx.h, self.h, ti, _ptr(pos), pos.size, C.byref(cnt)), "attn_read_selection")
        return None if cnt.value < 0 else pos[:cnt.value].copy()

    def decode(self, q, k, v, iq=None, ik=None):
        parts = [q, k, v] + ([iq, ik] if iq is not None else [])
        qkv = np.ascontiguousarray(np.concatenate(parts, axis=1), dtype=np.float32)
        t = qkv.shape[0]
        out = np.empty((t, self.nh * self.hd), dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_attn_decode_kv4(self.ctx.h, self.h, _ptr(qkv), t, _ptr(out)), "attn_decode_kv4")
        return out

    def close(self):
        if getattr(self, "h", None) and getattr(self.ctx, "h", None):
            self.ctx.L.pyre_attn_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class TensorDesc(C.Structure):
    _fields_ = [("ggml_type", C.c_uint32), ("on_device", C.c_uint32), ("rows", C.c_uint64), ("cols", C.c_uint64), ("data", C.c_void_p)]


class Gguf:
    """GGUF container reader (Gguf::open of the reference, gguf_q.rs:297-336); host only, needs no GPU."""

    def __init__(self, path):
        self.L = load()
        h = C.c_void_p(); err = C.create_string_buffer(1024)
        rc = self.L.pyre_gguf_open(os.fsencode(path), C.byref(h), err, len(err))
        if rc:
            raise PyreError("gguf_open: %s" % err.value.decode(errors="replace"))
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            self.L.pyre_gguf_close(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def n_shards(self):
        return self.L.pyre_gguf_n_shards(self.h)

    def names(self):
        return [self.L.pyre_gguf_tensor_name(self.h, i).decode() for i in range(self.L.pyre_gguf_n_tensors(self.h))]

    def has(self, name):
        return bool(self.L.pyre_gguf_has(self.h, name.encode()))

    def tensor(self, name):
        """(ggml type, rows, cols, stored shape, bytes as a numpy uint8 copy)"""
        from . import synth
        td = TensorDesc(); nd = C.c_uint32(); dims = (C.c_uint64 * 8)(); err = C.create_string_buffer(1024)
        rc = self.L.pyre_gguf_tensor(self.h, name.encode(), C.byref(td), C.byref(nd), dims, err, len(err))
        if rc:
            raise PyreError("gguf_tensor: %s" % err.value.decode(errors="replace"))
        el, bs, _ = synth.GEOM[td.ggml_type]
        nbytes = td.rows * (td.cols // el) * bs
        data = np.ctypeslib.as_array(C.cast(td.data, C.POINTER(C.c_uint8)), shape=(nbytes,)).copy()
        return td.ggml_type, td.rows, td.cols, tuple(dims[i] for i in range(nd.value)), data

    def u64(self, key, default=None):
        v = C.c_uint64()
        if self.L.pyre_gguf_meta_u64(self.h, key.encode(), C.byref(v)) == 0:
            return v.value
        if default is None:
            raise KeyError(key)
        return default

    def f64(self, key):
        v = C.c_double()
        if self.L.pyre_gguf_meta_f64(self.h, key.encode(), C.byref(v)) != 0:
            raise KeyError(key)
        return v.value

    def string(self, key):
        b = C.create_string_buffer(4096)
        if self.L.pyre_gguf_meta_str(self.h, key.encode(), b, len(b)) != 0:
            raise KeyError(key)
        return b.value.decode(errors="replace")

    def arr_u64(self, key):
        n = self.L.pyre_gguf_meta_arr_u64(self.h, key.encode(), None, 0)
        if n < 0:
            raise KeyError(key)
        out = (C.c_uint64 * max(n, 1))()
        self.L.pyre_gguf_meta_arr_u64(self.h, key.encode(), out, n)
        return [out[i] for i in range(n)]


class ModelCfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "d", "hc", "hc_lr", "n_head", "n_kv", "hd", "n_rot")] + \
               [("rope_base", C.c_float), ("eps", C.c_float)] + \
               [(n, C.c_int32) for n in ("n_exp", "top_k", "ff_exp", "lin_nk", "lin_nv", "lin_dk", "lin_dv", "conv_k",
                                         "full_every", "vocab", "kv_bits", "kv_recent", "idx_nh", "idx_hd", "idx_ratio", "idx_budget", "ctx_train", "ctx")] + \
               [(n, C.c_int32) for n in ("ple_ngram", "ple_per_gram", "ple_conv_k", "ple_dim")] + [("ple_eos", C.c_uint32), ("ple_reserved", C.c_int32),
                ("ple_mult", C.c_uint64 * 8), ("ple_off", C.c_uint64 * 16), ("ple_vocab", C.c_uint64 * 16)]


LAYER_SLOTS, GLOBAL_SLOTS = 41, 6


def fill_cfg(dst, src):
    """Copies the configuration fields of `src` (any object with the field names; PLE fields optional) into the ctypes struct."""
    for name, ty in dst._fields_:
        if name == "ple_reserved":
            continue
        v = getattr(src, name, 0)
        if name in ("ple_mult", "ple_off", "ple_vocab"):
            arr = getattr(dst, name)
            for i, x in enumerate(list(v or ())[:len(arr)]):
                arr[i] = int(x)
        else:
            setattr(dst, name, v)
    return dst


class Model:
    """Model::{load, new_state, forward, forward_multi, spec_keep} of the reference over device-resident weights."""

    def __init__(self, ctx, cfg, layer_tensors, globals_):
        """cfg: object with the ModelCfg field names; layer_tensors: per layer dict slot -> (ty, rows, cols, data) where
        data is a numpy uint8 array (host) or an int device pointer; globals_: dict slot -> the same."""
        self.ctx = ctx
        self.cfg = fill_cfg(ModelCfg(), cfg)
        keep = []

        def desc(e):
            if e is None:
                return TensorDesc(0, 0, 0, 0, None)
            ty, rows, cols, data = e
            if isinstance(data, np.ndarray):
                data = np.ascontiguousarray(data); keep.append(data)
                return TensorDesc(ty, 0, rows, cols, data.ctypes.data)
            return TensorDesc(ty, 1, rows, cols, int(data))
        lt = (TensorDesc * (self.cfg.n_layers * LAYER_SLOTS))(*[desc(layer_tensors[il].get(s)) for il in range(self.cfg.n_layers) for s in range(LAYER_SLOTS)])
        gl = (TensorDesc * GLOBAL_SLOTS)(*[desc(globals_.get(s)) for s in range(GLOBAL_SLOTS)])
        h = C.c_void_p()
        ctx.check(ctx.L.pyre_model_create(ctx.h, C.byref(self.cfg), lt, gl, C.byref(h)), "model_create")
        self.h = h
        self.vocab = self.cfg.vocab

    @classmethod
    def from_gguf(cls, ctx, path, kv_bits=4, kv_recent=1024, ctx_tokens=0):
        """Model::load: configuration and tensors straight from a qwen4exp GGUF file (or its shards)."""
        self = cls.__new__(cls)
        self.ctx = ctx
        h = C.c_void_p()
        ctx.check(ctx.L.pyre_model_load_gguf(ctx.h, os.fsencode(path), kv_bits, kv_recent, ctx_tokens, C.byref(h)), "model_load_gguf")
        self.h = h
        g = Gguf(path); a = "qwen4exp."
        c = ModelCfg()
        for field, key in (("n_layers", "block_count"), ("d", "embedding_length"), ("hc", "hyper_connection.count"), ("hc_lr", "hyper_connection.low_rank"),
                           ("n_head", "attention.head_count"), ("n_kv", "attention.head_count_kv"), ("hd", "attention.key_length"), ("n_rot", "rope.dimension_count"),
                           ("n_exp", "expert_count"), ("top_k", "expert_used_count"), ("ff_exp", "expert_feed_forward_length"), ("lin_nk", "ssm.group_count"),
                           ("lin_nv", "ssm.time_step_rank"), ("lin_dk", "ssm.state_size"), ("lin_dv", "ssm.state_size"), ("conv_k", "ssm.conv_kernel")):
            setattr(c, field, g.u64(a + key))
        c.full_every = g.u64(a + "full_attention_interval", 4)
        c.rope_base = g.f64(a + "rope.freq_base"); c.eps = g.f64(a + "attention.layer_norm_rms_epsilon")
        c.vocab = g.tensor("token_embd.weight")[3][1]; c.kv_bits = kv_bits; c.kv_recent = kv_recent
        c.idx_budget = g.u64(a + "attention.indexer.top_k", 2048); c.idx_hd = g.u64(a + "attention.indexer.key_length", 128)
        c.idx_nh = g.u64(a + "attention.indexer.head_count", 0) if g.has("blk.%d.indexer.q_proj.weight" % (c.full_every - 1)) else 0
        try:
            c.idx_ratio = max(max(g.arr_u64(a + "attention.compress_ratios") or [4]), 1)
        except KeyError:
            c.idx_ratio = 4
        c.ctx_train = g.u64(a + "context_length", 262144); c.ctx = ctx_tokens or c.ctx_train
        try:
            has_ple = bool(g.arr_u64(a + "ple.layers"))
        except KeyError:
            has_ple = False
        if has_ple:
            c.ple_ngram = g.u64(a + "ple.ngram_size", 0); c.ple_per_gram = g.u64(a + "ple.heads_per_ngram", 0); c.ple_conv_k = g.u64(a + "ple.conv_kernel", 0)
            c.ple_eos = g.u64(a + "ple.eos_token_id", 0); c.ple_dim = g.u64(a + "embedding_length_per_layer_input", 0)
        g.close()
        self.cfg = c; self.vocab = c.vocab
        return self

    @property
    def weight_bytes_per_token(self):
        return self.ctx.L.pyre_model_weight_bytes_per_token(self.h)

    def prompt_blocks(self):
        """Blocks of up to 1024 prompt tokens taken layer by layer with the FFN grouped by expert since the model was created."""
        return self.ctx.L.pyre_model_prompt_blocks(self.h)

    def new_state(self, max_ctx):
        return State(self, max_ctx)

    def forward(self, ids, st, want_logits=True):
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        lg = np.empty(self.vocab, dtype=np.float32) if want_logits else None
        self.ctx.check(self.ctx.L.pyre_forward(self.ctx.h, self.h, st.h, _ptr(ids), ids.size, _ptr(lg)), "forward")
        return lg

    def forward_multi(self, ids, st):
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        lg = np.empty((ids.size, self.vocab), dtype=np.float32)
        self.ctx.check(self.ctx.L.pyre_forward_multi(self.ctx.h, self.h, st.h, _ptr(ids), ids.size, _ptr(lg)), "forward_multi")
        return lg

    def spec_keep(self, st, t, keep):
        self.ctx.check(self.ctx.L.pyre_spec_keep(self.ctx.h, self.h, st.h, t, keep), "spec_keep")

    def generate_greedy(self, st, first_logits, n_out, n_draft=0, draft_stream=None):
        fl = np.ascontiguousarray(first_logits, dtype=np.float32)
        out = np.empty(n_out, dtype=np.uint32)
        ds = None
        if draft_stream is not None:
            ds = np.ascontiguousarray(draft_stream, dtype=np.uint32)
            assert ds.size >= n_out + 8
        rounds = C.c_int(0)
        self.ctx.check(self.ctx.L.pyre_generate_greedy(self.ctx.h, self.h, st.h, _ptr(fl), n_out, _ptr(out), n_draft, _ptr(ds), C.byref(rounds)), "generate_greedy")
        return out, rounds.value

    def generate_greedy_ngram(self, st, history, first_logits, n_out, k=4, ng_min=3, ng_max=8):
        """spec::generate (greedy) with the prompt-lookup drafter; returns (tokens, rounds, drafted, accepted)."""
        fl = np.ascontiguousarray(first_logits, dtype=np.float32); hs = np.ascontiguousarray(history, dtype=np.uint32)
        out = np.empty(n_out, dtype=np.uint32); r, d, a = C.c_int(0), C.c_int(0), C.c_int(0)
        self.ctx.check(self.ctx.L.pyre_generate_greedy_ngram(self.ctx.h, self.h, st.h, _ptr(hs), hs.size, _ptr(fl), n_out, _ptr(out), k, ng_min, ng_max,
                                                             C.byref(r), C.byref(d), C.byref(a)), "generate_greedy_ngram")
        return out, r.value, d.value, a.value

    def decode_greedy_dev(self, st, first, n_steps, fetch=True):
        out = np.empty(n_steps, dtype=np.uint32) if fetch else None
        self.ctx.check(self.ctx.L.pyre_decode_greedy_dev(self.ctx.h, self.h, st.h, int(first), n_steps, _ptr(out)), "decode_greedy_dev")
        return out

    def close(self):
        if getattr(self, "h", None) and getattr(self.ctx, "h", None):
            self.ctx.L.pyre_model_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


MTP_SLOTS = 30


class MtpCfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_exp", "top_k", "ff", "window", "n_draft_vocab")]


class Mtp:
    """The MTP drafter (src/model/mtp.rs) beside a Model: tensors is a dict slot -> (ty, rows, cols, data) over the
    PYRE_MTP_* slots, draft_ids the vocabulary ids of the draft head's rows."""

    def __init__(self, model, n_exp, top_k, ff, window, tensors, draft_ids):
        self.m = model; ctx = model.ctx
        ids = np.ascontiguousarray(draft_ids, dtype=np.uint32)
        self.cfg = MtpCfg(n_exp, top_k, ff, window, ids.size)
        keep = []

        def desc(e):
            if e is None:
                return TensorDesc(0, 0, 0, 0, None)
            ty, rows, cols, data = e
            if isinstance(data, np.ndarray):
                data = np.ascontiguousarray(data); keep.append(data)
                return TensorDesc(ty, 0, rows, cols, data.ctypes.data)
            return TensorDesc(ty, 1, rows, cols, int(data))
        ts = (TensorDesc * MTP_SLOTS)(*[desc(tensors.get(s)) for s in range(MTP_SLOTS)])
        h = C.c_void_p()
        ctx.check(ctx.L.pyre_mtp_create(ctx.h, model.h, C.byref(self.cfg), ts, _ptr(ids), C.byref(h)), "mtp_create")
        self.h = h

    @classmethod
    def from_safetensors(cls, model, path, draft_ids, top_k=0, window=0, head=None):
        """Mtp::load: the drafter from its one-file BF16 checkpoint; head = (ty, rows, cols, data) or None (rows of the
        main model's output matrix, f32)."""
        self = cls.__new__(cls); self.m = model; ctx = model.ctx
        ids = np.ascontiguousarray(draft_ids, dtype=np.uint32); hd = None; keep = None
        if head is not None:
            ty, rows, cols, data = head; keep = np.ascontiguousarray(data); hd = C.byref(TensorDesc(ty, 0, rows, cols, keep.ctypes.data))
        h = C.c_void_p()
        ctx.check(ctx.L.pyre_mtp_load_safetensors(ctx.h, model.h, os.fsencode(path), top_k, window, _ptr(ids), ids.size, hd, C.byref(h)), "mtp_load_safetensors")
        self.h = h; self.cfg = MtpCfg(0, top_k, 0, window or 128, ids.size)
        return self

    def attach(self, st):
        self.m.ctx.check(self.m.ctx.L.pyre_state_attach_mtp(self.m.ctx.h, st.h, self.h), "state_attach_mtp")

    def draft(self, st, pending, k, min_p=0.0):
        """Model::mtp_draft: (ids, probabilities) of up to k drafts after `pending`."""
        ids = np.zeros(8, dtype=np.uint32); ps = np.zeros(8, dtype=np.float32); n = C.c_int(0)
        self.m.ctx.check(self.m.ctx.L.pyre_mtp_draft(self.m.ctx.h, self.h, st.h, int(pending), k, min_p, _ptr(ids), _ptr(ps), C.byref(n)), "mtp_draft")
        return ids[:n.value].copy(), ps[:n.value].copy()

    def kv(self, st):
        """(first cell, K [n][n_kv*hd], V) of the drafter's cache."""
        c = self.m.cfg; row = c.n_kv * c.hd
        k = np.zeros((self.cfg.window + 8, row), dtype=np.float32); v = np.zeros_like(k); c0, n = C.c_int(0), C.c_int(0)
        self.m.ctx.check(self.m.ctx.L.pyre_mtp_read_kv(self.m.ctx.h, st.h, C.byref(c0), C.byref(n), _ptr(k), _ptr(v)), "mtp_read_kv")
        return c0.value, k[:n.value].copy(), v[:n.value].copy()

    def generate_greedy(self, st, first_logits, n_out, k=3, min_p=0.0):
        """spec::generate (greedy) with this drafter; returns (tokens, rounds, drafted, accepted)."""
        fl = np.ascontiguousarray(first_logits, dtype=np.float32)
        out = np.empty(n_out, dtype=np.uint32); r, d, a = C.c_int(0), C.c_int(0), C.c_int(0)
        self.m.ctx.check(self.m.ctx.L.pyre_generate_greedy_mtp(self.m.ctx.h, self.m.h, self.h, st.h, _ptr(fl), n_out, _ptr(out), k, min_p,
                                                               C.byref(r), C.byref(d), C.byref(a)), "generate_greedy_mtp")
        return out, r.value, d.value, a.value

    def generate_greedy_forced(self, st, first_logits, n_out, forced_stream, k=3):
        """The same loop with the drafter's ids replaced (after it ran) by forced_stream: the accepted path end to end."""
        fl = np.ascontiguousarray(first_logits, dtype=np.float32); fs = np.ascontiguousarray(forced_stream, dtype=np.uint32)
        assert fs.size >= n_out + 8
        out = np.empty(n_out, dtype=np.uint32); r, d, a = C.c_int(0), C.c_int(0), C.c_int(0)
        self.m.ctx.check(self.m.ctx.L.pyre_generate_greedy_mtp_forced(self.m.ctx.h, self.m.h, self.h, st.h, _ptr(fl), n_out, _ptr(out), k, _ptr(fs),
                                                                      C.byref(r), C.byref(d), C.byref(a)), "generate_greedy_mtp_forced")
        return out, r.value, d.value, a.value

    def close(self):
        if getattr(self, "h", None) and getattr(self.m, "h", None) and getattr(self.m.ctx, "h", None):
            self.m.ctx.L.pyre_mtp_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Snap:
    def __init__(self, ctx, h):
        self.ctx, self.h = ctx, h

    def __len__(self):
        return self.ctx.L.pyre_snap_len(self.h)

    @property
    def nbytes(self):
        return self.ctx.L.pyre_snap_bytes(self.h)

    def close(self):
        if getattr(self, "h", None) and getattr(self.ctx, "h", None):
            self.ctx.L.pyre_snap_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class State:
    def __init__(self, model, max_ctx):
        self.m = model
        h = C.c_void_p()
        model.ctx.check(model.ctx.L.pyre_state_create(model.ctx.h, model.h, max_ctx, C.byref(h)), "state_create")
        self.h = h

    def __len__(self):
        return self.m.ctx.L.pyre_state_len(self.h)

    def reset(self):
        self.m.ctx.check(self.m.ctx.L.pyre_state_reset(self.m.ctx.h, self.h), "state_reset")

    def gdn(self, li):
        c = self.m.cfg
        ch = 2 * c.lin_nk * c.lin_dk + c.lin_nv * c.lin_dv
        conv = np.empty(((c.conv_k - 1) * ch,), dtype=np.float32)
        ssm = np.empty((c.lin_nv * c.lin_dk * c.lin_dv,), dtype=np.float32)
        self.m.ctx.check(self.m.ctx.L.pyre_state_read_gdn(self.m.ctx.h, self.h, li, _ptr(conv), _ptr(ssm)), "state_read_gdn")
        return conv, ssm

    def ple_hist(self, pi):
        c = self.m.cfg
        h = np.empty(((c.ple_conv_k - 1) * c.ple_ngram, c.hc * c.d), dtype=np.float32)
        self.m.ctx.check(self.m.ctx.L.pyre_state_read_ple(self.m.ctx.h, self.h, pi, _ptr(h)), "state_read_ple")
        return h

    def kv(self, ai):
        c = self.m.cfg
        n = len(self)
        k = np.empty((n, c.n_kv * c.hd), dtype=np.float32); v = np.empty_like(k)
        self.m.ctx.check(self.m.ctx.L.pyre_state_read_kv(self.m.ctx.h, self.h, ai, _ptr(k), _ptr(v)), "state_read_kv")
        return k, v

    @property
    def capacity(self):
        return self.m.ctx.L.pyre_state_capacity(self.h)

    def snapshot(self):
        """Model::snapshot: (handle, length, bytes); hand the handle to restore() of any state of the same model."""
        h = C.c_void_p()
        self.m.ctx.check(self.m.ctx.L.pyre_state_snapshot(self.m.ctx.h, self.h, C.byref(h)), "state_snapshot")
        return Snap(self.m.ctx, h)

    def restore(self, snap):
        self.m.ctx.check(self.m.ctx.L.pyre_state_restore(self.m.ctx.h, self.h, snap.h), "state_restore")

    def close(self):
        if getattr(self, "h", None) and getattr(self.m, "h", None) and getattr(self.m.ctx, "h", None):      # never after its context
            self.m.ctx.L.pyre_state_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Session:
    """engine_qn::run of the reference (src/engine_qn.rs:92-170) over one resident state: chunk-grid prefill with a prefix
    cache of device-resident snapshots, then greedy generation."""

    def __init__(self, model, max_ctx, chunk=256, cache_bytes=3072 << 20):
        self.m = model; self.ctx = model.ctx
        h = C.c_void_p()
        self.ctx.check(self.ctx.L.pyre_session_create(self.ctx.h, model.h, max_ctx, chunk, cache_bytes, C.byref(h)), "session_create")
        self.h = h

    def prefill(self, prompt):
        """(logits after the prompt, prompt tokens not recomputed, whether they came from a snapshot)"""
        ids = np.ascontiguousarray(prompt, dtype=np.uint32)
        lg = np.empty(self.m.vocab, dtype=np.float32); cached = C.c_int32(); snap = C.c_int32()
        self.ctx.check(self.ctx.L.pyre_session_prefill(self.ctx.h, self.h, _ptr(ids), ids.size, _ptr(lg), C.byref(cached), C.byref(snap)), "session_prefill")
        return lg, cached.value, bool(snap.value)

    def generate_greedy(self, first_logits, n_out, n_draft=0, draft_stream=None):
        fl = np.ascontiguousarray(first_logits, dtype=np.float32); out = np.empty(n_out, dtype=np.uint32); rounds = C.c_int32()
        ds = np.ascontiguousarray(draft_stream, dtype=np.uint32) if draft_stream is not None else None
        self.ctx.check(self.ctx.L.pyre_session_generate_greedy(self.ctx.h, self.h, _ptr(fl), n_out, _ptr(out), n_draft, _ptr(ds) if ds is not None else None, C.byref(rounds)), "session_generate_greedy")
        return out, rounds.value

    def stats(self):
        """(snapshots held, their bytes, tokens the state has consumed, snapshot lengths oldest first)"""
        n = C.c_int32(); b = C.c_size_t(); ln = C.c_int32()
        self.ctx.L.pyre_session_stats(self.h, C.byref(n), C.byref(b), C.byref(ln))
        return n.value, b.value, ln.value, [self.ctx.L.pyre_session_snapshot_len(self.h, i) for i in range(n.value)]

    def close(self):
        if getattr(self, "h", None) and getattr(self.ctx, "h", None):
            self.ctx.L.pyre_session_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
