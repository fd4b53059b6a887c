"""ctypes binding of the CPU oracle (oracle/liborc.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")
_SO = os.path.join(_DIR, "liborc.so")

F32, F16, Q8_0, Q4_K, IQ2_XS, IQ3_S, BF16 = 0, 1, 8, 12, 17, 21, 30
Q4_0, Q5_0, Q6_K, IQ2_XXS, IQ3_XXS, IQ4_NL, IQ2_S, IQ4_XS, Q3_K, Q2_0, Q5_K, IQ1_M = 2, 6, 14, 16, 18, 20, 22, 23, 11, 42, 13, 29
(HCA_NORM, HCA_DOWN, HCA_INJECT, HCA_UP, HCF_NORM, HCF_DOWN, HCF_INJECT, HCF_UP, ATTN_Q, ATTN_K, ATTN_V, ATTN_O,
 ATTN_QN, ATTN_KN, LIN_QKV, LIN_Z, LIN_BETA, LIN_ALPHA, LIN_A, LIN_DT, LIN_CONV, LIN_NORM, LIN_OUT, ROUTER, GATE_E,
 UP_E, DOWN_E, SH_GATE_INP, SH_GATE, SH_UP, SH_DOWN, IDX_Q, IDX_K, IDX_QN, IDX_KN,
 PLE_KEY, PLE_VALUE, PLE_NK, PLE_NQ, PLE_NC, PLE_CONV, LAYER_SLOTS) = range(42)
G_EMBD, G_HEAD_NORM, G_HEAD_DOWN, G_HEAD_UP, G_OUT, G_PLE_TAB, GLOBAL_SLOTS = range(7)


class Tensor(C.Structure):
    _fields_ = [("ty", C.c_uint32), ("rows", C.c_uint64), ("cols", C.c_uint64), ("data", C.c_void_p)]


class Cfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "d", "hc", "hc_lr", "n_head", "n_kv", "hd", "n_rot")] + \
               [("rope_base", C.c_float), ("eps", C.c_float)] + \
               [(n, C.c_int32) for n in ("n_exp", "top_k", "ff_exp", "lin_nk", "lin_nv", "lin_dk", "lin_dv", "conv_k",
                                         "full_every", "vocab", "kv_bits", "kv_recent", "idx_nh", "idx_hd", "idx_ratio", "idx_budget", "ctx_train", "ctx")] + \
               [(n, C.c_int32) for n in ("ple_ngram", "ple_per_gram", "ple_conv_k", "ple_dim")] + [("ple_eos", C.c_uint32), ("ple_reserved", C.c_int32),
                ("ple_mult", C.c_uint64 * 8), ("ple_off", C.c_uint64 * 16), ("ple_vocab", C.c_uint64 * 16)]


def build():
    subprocess.check_call(["make", "-s", "-C", _DIR])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        L.orc_dot.restype = C.c_float
        L.orc_kv4_get.restype = C.c_float
        L.orc_kv_packed_boundary.restype = C.c_size_t
        L.orc_kv_packed_boundary.argtypes = [C.c_size_t, C.c_int, C.c_int]
        L.orc_argmax.restype = C.c_uint32
        L.orc_ksigns.restype = C.c_uint8
        for n in ("orc_sigm", "orc_silu", "orc_softplus"):
            getattr(L, n).restype = C.c_float
            getattr(L, n).argtypes = [C.c_float]
        L.orc_model_create.restype = C.c_void_p
        L.orc_state_create.restype = C.c_void_p
        L.orc_rope_inv_yarn.restype = C.c_float
        for n in ("orc_state_conv", "orc_state_ssm", "orc_state_k", "orc_state_v", "orc_state_ik", "orc_state_ib", "orc_state_ple_hist"):
            getattr(L, n).restype = C.POINTER(C.c_float)
        L.orc_mtp_create.restype = C.c_void_p
        L.orc_mtp_r.restype = C.POINTER(C.c_float)
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def dequant(ty, raw, n):
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    y = np.empty(n, dtype=np.float32)
    rc = lib().orc_dequant(C.c_uint32(ty), _p(raw), C.c_size_t(n), _p(y))
    assert rc == 0
    return y


def dot(a, b):
    a, b = f32(a), f32(b)
    return float(lib().orc_dot(_p(a), _p(b), C.c_size_t(a.size)))


def matmul(ty, raw, rows, cols, x, threads=4):
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    x = f32(x).reshape(-1, cols)
    t = x.shape[0]
    y = np.empty((t, rows), dtype=np.float32)
    rc = lib().orc_matmul(C.c_uint32(ty), _p(raw), C.c_size_t(rows), C.c_size_t(cols), _p(x), C.c_int(t), _p(y), C.c_int(threads))
    assert rc == 0
    return y


def kv4_pack(x):
    x = f32(x).reshape(-1)
    w = np.empty(x.size // 8, dtype=np.uint32)
    sc = np.empty(x.size // 32, dtype=np.float32)
    lib().orc_kv4_pack(_p(x), C.c_size_t(x.size), _p(w), _p(sc))
    return w, sc


def kv4_unpack(w, sc, n):
    return np.array([lib().orc_kv4_get(_p(w), _p(sc), C.c_size_t(i)) for i in range(n)], dtype=np.float32)


def kvq_roundtrip(x, bits):
    y = f32(x).reshape(-1).copy()
    lib().orc_kvq_roundtrip(_p(y), C.c_size_t(y.size), C.c_int(bits))
    return y.reshape(np.shape(x))


def packed_boundary(n, kv_bits=4, recent=1024):
    return int(lib().orc_kv_packed_boundary(n, kv_bits, recent))


def rope_inv(n_rot, base):
    inv = np.empty(n_rot // 2, dtype=np.float32)
    lib().orc_rope_inv(C.c_int(n_rot), C.c_float(base), _p(inv))
    return inv


def argmax(l):
    l = f32(l)
    return int(lib().orc_argmax(_p(l), C.c_size_t(l.size)))


def top_k(r, k):
    r = f32(r)
    idx = np.empty(k, dtype=np.int32)
    w = np.empty(k, dtype=np.float32)
    rc = lib().orc_top_k(_p(r), C.c_int(r.size), C.c_int(k), _p(idx), _p(w))
    assert rc == 0
    return idx, w


def tensor(ty, rows, cols, arr):
    """arr: numpy array holding the raw bytes (kept alive by the caller)."""
    return Tensor(ty, rows, cols, arr.ctypes.data if arr is not None else None)


def vec_tensor(arr):
    return Tensor(F32, 1, arr.size, arr.ctypes.data)


def gdn_core(nk, nv, dk, dv, conv_k, eps, a, dt, conv_w, norm_w, qkv, z, beta, alpha, conv_state, ssm):
    """Runs t tokens; conv_state and ssm (float32 arrays) are updated in place. Returns out [t][nv*dv]."""
    qkv = f32(qkv); t = qkv.shape[0]
    z, beta, alpha = f32(z), f32(beta), f32(alpha)
    a, dt, conv_w, norm_w = f32(a), f32(dt), f32(conv_w), f32(norm_w)
    out = np.empty((t, nv * dv), dtype=np.float32)
    lib().orc_gdn_core(nk, nv, dk, dv, conv_k, C.c_float(eps), _p(a), _p(dt), _p(conv_w), _p(norm_w), _p(qkv), _p(z), _p(beta), _p(alpha),
                       C.c_int(t), _p(conv_state), _p(ssm), _p(out))
    return out


def attn_core(nh, nkv, hd, n_rot, eps, inv, qn, kn, q, k, v, start, kv_bits, kv_recent, kc, vc):
    q = f32(q); t = q.shape[0]
    k, v, qn, kn, inv = f32(k), f32(v), f32(qn), f32(kn), f32(inv)
    out = np.empty((t, nh * hd), dtype=np.float32)
    lib().orc_attn_core(nh, nkv, hd, n_rot, C.c_float(eps), _p(inv), _p(qn), _p(kn), _p(q), _p(k), _p(v), C.c_int(start), C.c_int(t),
                        C.c_int(kv_bits), C.c_int(kv_recent), _p(kc), _p(vc), _p(out))
    return out


def rope_inv_yarn(n_rot, base, ctx_train, ctx):
    inv = np.empty(n_rot // 2, dtype=np.float32)
    ms = lib().orc_rope_inv_yarn(C.c_int(n_rot), C.c_float(base), C.c_int(ctx_train), C.c_int(ctx), _p(inv))
    return inv, float(ms)


def attn_core_qsa(nh, nkv, hd, n_rot, eps, inv, mscale, qn, kn, q, k, v, start, kv_bits, kv_recent, kc, vc,
                  idx_nh, idx_hd, idx_ratio, idx_budget, iqn, ikn, iq, ik, ikc, ibc):
    """Returns (out [t][nh*hd], [positions or None per token]); the caches kc, vc, ikc, ibc are updated in place."""
    q = f32(q); t = q.shape[0]
    k, v, qn, kn, inv, iqn, ikn, iq, ik = (f32(a) for a in (k, v, qn, kn, inv, iqn, ikn, iq, ik))
    out = np.empty((t, nh * hd), dtype=np.float32)
    stride = idx_budget + 2 * idx_ratio
    sel = np.zeros((t, stride), dtype=np.int32); sel_n = np.zeros(t, dtype=np.int32)
    lib().orc_attn_core_qsa(nh, nkv, hd, n_rot, C.c_float(eps), _p(inv), C.c_float(mscale), _p(qn), _p(kn), _p(q), _p(k), _p(v), C.c_int(start), C.c_int(t),
                            C.c_int(kv_bits), C.c_int(kv_recent), _p(kc), _p(vc), C.c_int(idx_nh), C.c_int(idx_hd), C.c_int(idx_ratio), C.c_int(idx_budget),
                            _p(iqn), _p(ikn), _p(iq), _p(ik), _p(ikc), _p(ibc), _p(out), _p(sel), _p(sel_n), C.c_int(stride))
    return out, [None if sel_n[i] < 0 else sel[i, :sel_n[i]].copy() for i in range(t)]


def moe_ffn(d, n_exp, k, ff, router, gate_e, up_e, down_e, sh_gate_inp, sh_gate, sh_up, sh_down, x, threads=4):
    x = f32(x).reshape(-1, d); t = x.shape[0]
    y = np.empty((t, d), dtype=np.float32)
    idx = np.empty((t, k), dtype=np.int32); w = np.empty((t, k), dtype=np.float32)
    sgi = f32(sh_gate_inp)
    rc = lib().orc_moe_ffn(d, n_exp, k, ff, C.byref(router), C.byref(gate_e), C.byref(up_e), C.byref(down_e), _p(sgi),
                           C.byref(sh_gate), C.byref(sh_up), C.byref(sh_down), _p(x), C.c_int(t), _p(y), _p(idx), _p(w), C.c_int(threads))
    assert rc == 0
    return y, idx, w


def hc_mix(d, hc, eps, norm, down, inject, up, x, threads=4):
    x = f32(x).reshape(-1, hc * d); t = x.shape[0]
    norm = f32(norm)
    mixed = np.empty((t, d), dtype=np.float32); inj = np.empty((t, hc), dtype=np.float32)
    rc = lib().orc_hc_mix(d, hc, C.c_float(eps), _p(norm), C.byref(down), C.byref(inject) if inject is not None else None, C.byref(up),
                          _p(x), C.c_int(t), _p(mixed), _p(inj), C.c_int(threads))
    assert rc == 0
    return mixed, inj


def hc_combine(d, hc, x, out, inj):
    x = f32(x).copy(); out = f32(out); inj = f32(inj)
    t = x.size // (hc * d)
    lib().orc_hc_combine(d, hc, _p(x), _p(out), _p(inj), C.c_int(t))
    return x


def ple_rows(cfg, tab, tokens, start, t):
    """cfg: orc.Cfg with the ple_* fields; tab: orc.Tensor; tokens: the history (uint32).  Returns emb [t][heads*dim]."""
    tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
    emb = np.empty((t, (cfg.ple_ngram - 1) * cfg.ple_per_gram * cfg.ple_dim), dtype=np.float32)
    rc = lib().orc_ple_rows(C.byref(cfg), C.byref(tab), _p(tokens), C.c_int(start), C.c_int(t), _p(emb))
    assert rc == 0, rc
    return emb


def ple(cfg, key, value, nk, nq, nc, conv, hist, emb, x, threads=2):
    """One PLE layer on t tokens: returns the updated x [t][hc*d]; hist [(conv_k-1)*ngram][hc*d] is advanced in place."""
    x = f32(x).copy().reshape(-1, cfg.hc * cfg.d); t = x.shape[0]
    nk, nq, nc, conv, emb = f32(nk), f32(nq), f32(nc), f32(conv), f32(emb)
    assert hist.dtype == np.float32 and hist.flags.c_contiguous
    rc = lib().orc_ple(C.byref(cfg), C.byref(key), C.byref(value), _p(nk), _p(nq), _p(nc), _p(conv), _p(hist), _p(emb), _p(x), C.c_int(t), C.c_int(threads))
    assert rc == 0, rc
    return x


class Model:
    """Oracle model over a weight set (see tests/modelgen.py for the container)."""

    def __init__(self, cfg, layer_tensors, globals_, threads=4, keep=()):
        self.cfg = cfg
        self._keep = keep
        n = cfg.n_layers * LAYER_SLOTS
        self._lt = (Tensor * n)(*layer_tensors)
        self._g = (Tensor * GLOBAL_SLOTS)(*globals_)
        self.h = C.c_void_p(lib().orc_model_create(C.byref(cfg), self._lt, self._g, C.c_int(threads)))
        assert self.h

    def new_state(self):
        return State(self)

    def forward(self, ids, st):
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        lg = np.empty(self.cfg.vocab, dtype=np.float32)
        rc = lib().orc_forward(self.h, st.h, _p(ids), C.c_int(ids.size), _p(lg))
        assert rc == 0, rc
        return lg

    def forward_multi(self, ids, st):
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        lg = np.empty((ids.size, self.cfg.vocab), dtype=np.float32)
        rc = lib().orc_forward_multi(self.h, st.h, _p(ids), C.c_int(ids.size), _p(lg))
        assert rc == 0, rc
        return lg

    def spec_keep(self, st, t, keep):
        assert lib().orc_spec_keep(self.h, st.h, C.c_int(t), C.c_int(keep)) == 0

    def generate_greedy(self, st, first_logits, n_out, n_draft=0, draft_stream=None):
        out = np.empty(n_out, dtype=np.uint32)
        fl = f32(first_logits)
        ds = None
        if draft_stream is not None:
            ds = np.ascontiguousarray(draft_stream, dtype=np.uint32)
            assert ds.size >= n_out + 8
        rounds = lib().orc_generate_greedy(self.h, st.h, _p(fl), C.c_int(n_out), _p(out), C.c_int(n_draft), _p(ds) if ds is not None else None)
        assert rounds >= 0
        return out, rounds

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_model_destroy(self.h)
            self.h = None


MTP_SLOTS = 30


class MtpCfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_exp", "top_k", "ff", "window", "n_draft_vocab")]


class Mtp:
    """The oracle's MTP drafter beside a Model; tensors: list of MTP_SLOTS orc.Tensor, draft_ids: uint32 ids of the head's rows."""

    def __init__(self, model, n_exp, top_k, ff, window, tensors, draft_ids, keep=()):
        self.m = model; self._keep = keep
        self.ids = np.ascontiguousarray(draft_ids, dtype=np.uint32)
        self.cfg = MtpCfg(n_exp, top_k, ff, window, self.ids.size)
        self._t = (Tensor * MTP_SLOTS)(*tensors)
        self.h = C.c_void_p(lib().orc_mtp_create(model.h, C.byref(self.cfg), self._t, _p(self.ids)))
        assert self.h

    def attach(self, st):
        lib().orc_state_attach_mtp(st.h, self.h)

    def draft(self, st, pending, k, min_p=0.0):
        ids = np.zeros(8, dtype=np.uint32); ps = np.zeros(8, dtype=np.float32)
        n = lib().orc_mtp_draft(self.h, self.m.h, st.h, C.c_uint32(int(pending)), C.c_int(k), C.c_float(min_p), _p(ids), _p(ps))
        assert n >= 0
        return ids[:n].copy(), ps[:n].copy()

    def kv(self, st):
        c = self.m.cfg; row = c.n_kv * c.hd
        c0 = C.c_int(0); k = C.POINTER(C.c_float)(); v = C.POINTER(C.c_float)()
        n = lib().orc_mtp_kv(st.h, C.byref(c0), C.byref(k), C.byref(v))
        if n == 0:
            return c0.value, np.zeros((0, row), np.float32), np.zeros((0, row), np.float32)
        return c0.value, np.ctypeslib.as_array(k, shape=(n, row)).copy(), np.ctypeslib.as_array(v, shape=(n, row)).copy()

    def residual(self, st, pos):
        c = self.m.cfg
        p = lib().orc_mtp_r(st.h, C.c_int(pos))
        return np.ctypeslib.as_array(p, shape=(c.hc * c.d,)).copy() if p else None

    def generate_greedy(self, st, first_logits, n_out, k=3, min_p=0.0):
        out = np.empty(n_out, dtype=np.uint32); fl = f32(first_logits); d, a = C.c_int(0), C.c_int(0)
        rc = lib().orc_generate_greedy_mtp(self.m.h, self.h, st.h, _p(fl), C.c_int(n_out), _p(out), C.c_int(k), C.c_float(min_p), C.byref(d), C.byref(a))
        assert rc == 0
        return out, d.value, a.value

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_mtp_destroy(self.h)
            self.h = None


class State:
    def __init__(self, model):
        self.m = model
        self.h = C.c_void_p(lib().orc_state_create(model.h))

    def __len__(self):
        return lib().orc_state_len(self.h)

    def ssm(self, li):
        c = self.m.cfg
        n = c.lin_nv * c.lin_dk * c.lin_dv
        return np.ctypeslib.as_array(lib().orc_state_ssm(self.h, li), shape=(n,))

    def conv(self, li):
        c = self.m.cfg
        ch = 2 * c.lin_nk * c.lin_dk + c.lin_nv * c.lin_dv
        return np.ctypeslib.as_array(lib().orc_state_conv(self.h, li), shape=((c.conv_k - 1) * ch,))

    def ple_hist(self, pi):
        c = self.m.cfg
        return np.ctypeslib.as_array(lib().orc_state_ple_hist(self.h, pi), shape=((c.ple_conv_k - 1) * c.ple_ngram, c.hc * c.d))

    def kcache(self, ai):
        c = self.m.cfg
        return np.ctypeslib.as_array(lib().orc_state_k(self.h, ai), shape=(len(self) * c.n_kv * c.hd,))

    def vcache(self, ai):
        c = self.m.cfg
        return np.ctypeslib.as_array(lib().orc_state_v(self.h, ai), shape=(len(self) * c.n_kv * c.hd,))

    def ikeys(self, ai):
        return np.ctypeslib.as_array(lib().orc_state_ik(self.h, ai), shape=(len(self) * self.m.cfg.idx_hd,))

    def iblocks(self, ai):
        c = self.m.cfg
        return np.ctypeslib.as_array(lib().orc_state_ib(self.h, ai), shape=((len(self) // max(c.idx_ratio, 1)) * c.idx_hd,))

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_state_destroy(self.h)
            self.h = None
