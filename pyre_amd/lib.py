"""ctypes binding of libpyre_hip.so (include/pyre_hip.h) plus thin host-side mirrors of the reference's types:
QMat (src/model/gguf_q.rs:201-247).  There is no CPU fallback: a missing library or a failing call raises."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libpyre_hip.so")

F32, F16, Q8_0, Q4_K, IQ2_XS, IQ3_S, BF16 = 0, 1, 8, 12, 17, 21, 30

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
        "pyre_qmat_dequant": (i32, [vp, vp, vp]),
        "pyre_qmat_dequant_dev": (i32, [vp, vp, vp]),
        "pyre_qmat_row": (i32, [vp, vp, sz, vp]),
        "pyre_qmatmul": (i32, [vp, vp, vp, i32, vp]),
        "pyre_qmatmul_dev": (i32, [vp, vp, vp, i32, vp]),
        "pyre_synth_blocks": (i32, [vp, u32, sz, u64, f32, f32, vp]),
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

    def matmul_dev(self, x_dev, t, y_dev):
        self.ctx.check(self.ctx.L.pyre_qmatmul_dev(self.ctx.h, self.h, _ptr(x_dev), t, _ptr(y_dev)), "qmatmul_dev")

    def close(self):
        if getattr(self, "h", None) and getattr(self.ctx, "h", None):
            self.ctx.L.pyre_qmat_destroy(self.h)
        self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
