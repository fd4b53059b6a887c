"""Synthetic qwen4exp weight sets (host side) for tests, smoke and the benchmark.

Tensor slots follow the GGUF tensor names the reference loads (qwen4exp_gguf.rs:494-512); the slot numbering is the
one include/pyre_hip.h declares.  Every tensor is (ggml type id, rows, cols, raw bytes) with rows = prod(shape[1:]),
cols = shape[0] as Gguf::mat lays them out (gguf_q.rs:326-331).
"""
from dataclasses import dataclass, field

import numpy as np

from . import synth

(HCA_NORM, HCA_DOWN, HCA_INJECT, HCA_UP, HCF_NORM, HCF_DOWN, HCF_INJECT, HCF_UP, ATTN_Q, ATTN_K, ATTN_V, ATTN_O,
 ATTN_QN, ATTN_KN, LIN_QKV, LIN_Z, LIN_BETA, LIN_ALPHA, LIN_A, LIN_DT, LIN_CONV, LIN_NORM, LIN_OUT, ROUTER, GATE_E,
 UP_E, DOWN_E, SH_GATE_INP, SH_GATE, SH_UP, SH_DOWN, IDX_Q, IDX_K, IDX_QN, IDX_KN,
 PLE_KEY, PLE_VALUE, PLE_NK, PLE_NQ, PLE_NC, PLE_CONV, LAYER_SLOTS) = range(42)
G_EMBD, G_HEAD_NORM, G_HEAD_DOWN, G_HEAD_UP, G_OUT, G_PLE_TAB, GLOBAL_SLOTS = range(7)

CFG_FIELDS = ("n_layers", "d", "hc", "hc_lr", "n_head", "n_kv", "hd", "n_rot", "rope_base", "eps", "n_exp", "top_k",
              "ff_exp", "lin_nk", "lin_nv", "lin_dk", "lin_dv", "conv_k", "full_every", "vocab", "kv_bits", "kv_recent",
              "idx_nh", "idx_hd", "idx_ratio", "idx_budget", "ctx_train", "ctx",
              "ple_ngram", "ple_per_gram", "ple_conv_k", "ple_dim", "ple_eos", "ple_mult", "ple_off", "ple_vocab")


@dataclass
class Config:
    n_layers: int = 4
    d: int = 256
    hc: int = 2
    hc_lr: int = 32
    n_head: int = 4
    n_kv: int = 2
    hd: int = 256
    n_rot: int = 64
    rope_base: float = 1e7
    eps: float = 1e-6
    n_exp: int = 8
    top_k: int = 2
    ff_exp: int = 256
    lin_nk: int = 2
    lin_nv: int = 4
    lin_dk: int = 128
    lin_dv: int = 128
    conv_k: int = 4
    full_every: int = 4
    vocab: int = 512
    kv_bits: int = 4
    kv_recent: int = 1024
    idx_nh: int = 0                   # QSA sparse indexer heads (0 = no indexer), key length, block size, token budget
    idx_hd: int = 128
    idx_ratio: int = 4
    idx_budget: int = 2048
    ctx_train: int = 0                # trained context and the context the model is built for (ctx > ctx_train > 0: YaRN)
    ctx: int = 0
    # per-layer n-gram embeddings (PLE): n-gram length (0 = none), table heads per length, conv kernel, table row width,
    # the token that cuts a context, hash multipliers per n-gram position, per head table offset and modulus; ple_layers
    # lists the layers that carry the ple_* tensors (see with_ple)
    ple_ngram: int = 0
    ple_per_gram: int = 0
    ple_conv_k: int = 0
    ple_dim: int = 0
    ple_eos: int = 0
    ple_mult: tuple = ()
    ple_off: tuple = ()
    ple_vocab: tuple = ()
    ple_layers: tuple = ()
    ple_type: int = synth.Q8_0        # type of per_layer_token_embd and of ple_key / ple_value
    # generation knobs (not part of the model contract)
    qtype: int = synth.IQ3_S          # type of every projection / expert / embedding / head matrix
    hc_type: int = synth.BF16         # type of the hyper-connection matrices (BF16 in real files)
    ff_sh: int = 0                    # shared-expert width (0 = ff_exp)
    d_lo: float = 1e-3
    d_hi: float = 2e-2
    # quantized hyper-connection matrices use a smaller scale range: with d in [1e-3, 2e-2] their gate pre-activations
    # reach the hundreds, every sigmoid saturates and the network becomes chaotic in f32 (f32 and f64 evaluations of
    # the same weights then differ by percents), which would make any parity statement meaningless
    hc_d_div: float = 64.0
    router_type: int = synth.BF16         # ffn_gate_inp: bf16, f32 or f16

    @property
    def ch(self):
        return 2 * self.lin_nk * self.lin_dk + self.lin_nv * self.lin_dv

    def full(self, il):
        return (il + 1) % self.full_every == 0


def a3b_config(**kw):
    """The Qwen-Next-style A3B hybrid of the benchmark: 48 layers (3 Gated DeltaNet + 1 gated attention per group),
    512 routed experts top-10 + 1 shared, d 2048, expert ff 512, vocab 151936, 4 hyper-connection streams."""
    c = Config(n_layers=48, d=2048, hc=4, hc_lr=256, n_head=16, n_kv=2, hd=256, n_rot=64, rope_base=1e7, eps=1e-6,
               n_exp=512, top_k=10, ff_exp=512, lin_nk=16, lin_nv=32, lin_dk=128, lin_dv=128, conv_k=4, full_every=4,
               vocab=151936, kv_bits=4, kv_recent=1024, qtype=synth.IQ3_S, hc_type=synth.IQ3_S)
    for k, v in kw.items():
        setattr(c, k, v)
    return c


def with_ple(c: Config, layers=(0, 2), ngram=3, per_gram=2, conv_k=3, dim=64, eos=7, sizes=(97, 131, 61, 251)):
    """Switches PLE on for `layers`: (ngram - 1) * per_gram heads with the given table sizes (cycled), stacked in one table."""
    nh = (ngram - 1) * per_gram
    vocab = [sizes[i % len(sizes)] + 2 * i for i in range(nh)]
    off = [sum(vocab[:i]) for i in range(nh)]
    mult = [(0x9E3779B97F4A7C15 * (2 * i + 1) + 0x1234567 * i) & 0xFFFFFFFFFFFFFFFF | 1 for i in range(ngram)]
    c.ple_ngram, c.ple_per_gram, c.ple_conv_k, c.ple_dim, c.ple_eos = ngram, per_gram, conv_k, dim, eos
    c.ple_mult, c.ple_off, c.ple_vocab, c.ple_layers = tuple(mult), tuple(off), tuple(vocab), tuple(layers)
    return c


def tensor_specs(c: Config):
    """[(layer or -1, slot, kind, ty, rows, cols)] for every tensor of the model; kind in {'q','vec:<name>'}."""
    sf = c.ff_sh or c.ff_exp
    w = c.hc * c.d
    out = []
    for il in range(c.n_layers):
        for base in (HCA_NORM, HCF_NORM):
            out += [(il, base, "vec:norm1", synth.F32, 1, w), (il, base + 1, "q", c.hc_type, c.hc_lr, w),
                    (il, base + 2, "q", c.hc_type, c.hc, w),
                    (il, base + 3, "q", c.hc_type, w, c.hc_lr)]
        if il in c.ple_layers:
            ein = (c.ple_ngram - 1) * c.ple_per_gram * c.ple_dim
            out += [(il, PLE_KEY, "q", c.ple_type, w, ein), (il, PLE_VALUE, "q", c.ple_type, c.d, ein), (il, PLE_NK, "vec:norm1", synth.F32, 1, w),
                    (il, PLE_NQ, "vec:norm1", synth.F32, 1, w), (il, PLE_NC, "vec:norm1", synth.F32, 1, w), (il, PLE_CONV, "vec:conv", synth.F32, 1, w * c.ple_conv_k)]
        if c.full(il):
            out += [(il, ATTN_Q, "q", c.qtype, c.n_head * 2 * c.hd, c.d), (il, ATTN_K, "q", c.qtype, c.n_kv * c.hd, c.d),
                    (il, ATTN_V, "q", c.qtype, c.n_kv * c.hd, c.d), (il, ATTN_O, "q", c.qtype, c.d, c.n_head * c.hd),
                    (il, ATTN_QN, "vec:norm1", synth.F32, 1, c.hd), (il, ATTN_KN, "vec:norm1", synth.F32, 1, c.hd)]
            if c.idx_nh > 0:
                out += [(il, IDX_Q, "q", c.qtype, c.idx_nh * c.idx_hd, c.d), (il, IDX_K, "q", c.qtype, c.idx_hd, c.d),
                        (il, IDX_QN, "vec:norm1", synth.F32, 1, c.idx_hd), (il, IDX_KN, "vec:norm1", synth.F32, 1, c.idx_hd)]
        else:
            out += [(il, LIN_QKV, "q", c.qtype, c.ch, c.d), (il, LIN_Z, "q", c.qtype, c.lin_nv * c.lin_dv, c.d),
                    (il, LIN_BETA, "q", c.qtype, c.lin_nv, c.d), (il, LIN_ALPHA, "q", c.qtype, c.lin_nv, c.d),
                    (il, LIN_A, "vec:a", synth.F32, 1, c.lin_nv), (il, LIN_DT, "vec:dt", synth.F32, 1, c.lin_nv),
                    (il, LIN_CONV, "vec:conv", synth.F32, 1, c.ch * c.conv_k), (il, LIN_NORM, "vec:norm1", synth.F32, 1, c.lin_dv),
                    (il, LIN_OUT, "q", c.qtype, c.d, c.lin_nv * c.lin_dv)]
        out += [(il, ROUTER, "router", c.router_type, c.n_exp, c.d), (il, GATE_E, "q", c.qtype, c.n_exp * c.ff_exp, c.d),
                (il, UP_E, "q", c.qtype, c.n_exp * c.ff_exp, c.d), (il, DOWN_E, "q", c.qtype, c.n_exp * c.d, c.ff_exp),
                (il, SH_GATE_INP, "vec:small", synth.F32, 1, c.d), (il, SH_GATE, "q", c.qtype, sf, c.d),
                (il, SH_UP, "q", c.qtype, sf, c.d), (il, SH_DOWN, "q", c.qtype, c.d, sf)]
    out += [(-1, G_EMBD, "q", c.qtype, c.vocab, c.d), (-1, G_HEAD_NORM, "vec:norm1", synth.F32, 1, w),
            (-1, G_HEAD_DOWN, "q", c.hc_type, c.hc_lr, w), (-1, G_HEAD_UP, "q", c.hc_type, w, c.hc_lr),
            (-1, G_OUT, "q", c.qtype, c.vocab, c.d)]
    if c.ple_layers:
        nh = (c.ple_ngram - 1) * c.ple_per_gram
        out += [(-1, G_PLE_TAB, "q", c.ple_type, max(c.ple_off[h] + c.ple_vocab[h] for h in range(nh)), c.ple_dim)]
    return out


def tensor_seed(seed, il, slot):
    return (seed * 1000003 + (il + 1) * 64 + slot) & 0x7FFFFFFFFFFFFFFF


HC_SLOTS_LAYER = (HCA_DOWN, HCA_INJECT, HCA_UP, HCF_DOWN, HCF_INJECT, HCF_UP)
HC_SLOTS_GLOBAL = (G_HEAD_DOWN, G_HEAD_UP)


# Random payloads of these two types decode to values about ten times larger per unit of the f16 scale than the others
# (6-bit value x int8 sub-scale; 6-bit sub-scale x level up to 127): their scale range shrinks by that factor so that a
# synthetic model has weights of the same size whatever type it is stored in.
WIDE_TYPES = {synth.Q6_K: 10.0, synth.IQ4_XS: 9.0}


def scale_range(c: Config, il, slot, ty=None):
    hc = slot in (HC_SLOTS_LAYER if il >= 0 else HC_SLOTS_GLOBAL)
    div = (c.hc_d_div if hc else 1.0) * WIDE_TYPES.get(ty, 1.0)
    return (c.d_lo / div, c.d_hi / div)


def host_tensor(c: Config, seed, il, slot, kind, ty, rows, cols):
    s = tensor_seed(seed, il, slot)
    if kind == "q":
        if ty in (synth.F32, synth.F16, synth.BF16):
            std = 1.0 / np.sqrt(cols)
            if ty == synth.BF16:
                return synth.bf16_normal(rows, cols, s, std)
            x = synth.normal((rows, cols), s, std)
            return (x if ty == synth.F32 else x.astype(np.float16)).view(np.uint8).reshape(-1).copy()
        return synth.matrix(ty, rows, cols, s, *scale_range(c, il, slot, ty))
    if kind == "router":
        if ty == synth.BF16:
            return synth.bf16_normal(rows, cols, s, 0.02)
        x = synth.normal((rows, cols), s, 0.02)
        return (x if ty == synth.F32 else x.astype(np.float16)).view(np.uint8).reshape(-1).copy()
    name = kind.split(":")[1]
    if name == "norm1":
        v = synth.normal((cols,), s, 0.1, 1.0)
    elif name == "a":
        v = -np.exp(synth.uniform((cols,), s, 0.0, float(np.log(16.0))))      # ssm_a = -exp(A_log), A_log ~ U(0, ln 16)
    elif name == "dt":
        v = np.zeros(cols, dtype=np.float32)
    elif name == "conv":
        v = synth.normal((cols,), s, 0.5)
    elif name == "small":
        v = synth.normal((cols,), s, 0.02)
    else:
        raise ValueError(kind)
    return v.astype(np.float32).view(np.uint8).reshape(-1).copy()


@dataclass
class HostWeights:
    cfg: Config
    seed: int
    layers: list = field(default_factory=list)     # per layer: dict slot -> (ty, rows, cols, bytes)
    globals_: dict = field(default_factory=dict)

    def f32(self, il, slot):
        ty, rows, cols, b = (self.layers[il] if il >= 0 else self.globals_)[slot]
        assert ty == synth.F32
        return b.view(np.float32)


def build_host(c: Config, seed=1):
    """All tensors as numpy byte arrays (only sensible for small configurations)."""
    hw = HostWeights(c, seed, [dict() for _ in range(c.n_layers)], {})
    for il, slot, kind, ty, rows, cols in tensor_specs(c):
        b = host_tensor(c, seed, il, slot, kind, ty, rows, cols)
        (hw.layers[il] if il >= 0 else hw.globals_)[slot] = (ty, rows, cols, b)
    return hw


def build_device(ctx, c: Config, seed=1):
    """The same tensors as build_host, with every quantized matrix generated on the device (pyre_synth_blocks is
    bit-identical to synth.blocks).  Returns (layers, globals, raw_device_buffers); the raw buffers can be freed once
    the model has been created."""
    layers = [dict() for _ in range(c.n_layers)]
    globals_ = {}
    raw = []
    for il, slot, kind, ty, rows, cols in tensor_specs(c):
        if kind == "q" and ty not in (synth.F32, synth.F16, synth.BF16):
            el, bs, _ = synth.GEOM[ty]
            nb = rows * (cols // el)
            dev = ctx.alloc(nb * bs)
            lo, hi = scale_range(c, il, slot, ty)
            ctx.synth_blocks(ty, nb, tensor_seed(seed, il, slot), lo, hi, dev_out=dev)
            raw.append(dev)
            entry = (ty, rows, cols, dev)
        else:
            entry = (ty, rows, cols, host_tensor(c, seed, il, slot, kind, ty, rows, cols))
        (layers[il] if il >= 0 else globals_)[slot] = entry
    return layers, globals_, raw


# ---- the MTP drafter's tensors (slots of include/pyre_hip.h's PYRE_MTP_* enum; names of src/model/mtp.rs:99-117) -----------
(MTP_PRE_E, MTP_PRE_H, MTP_FC_E, MTP_FC_H, MTP_HCA_NORM, MTP_HCA_DOWN, MTP_HCA_INJECT, MTP_HCA_UP, MTP_HCF_NORM, MTP_HCF_DOWN,
 MTP_HCF_INJECT, MTP_HCF_UP, MTP_MIX_NORM, MTP_MIX_DOWN, MTP_MIX_UP, MTP_Q, MTP_K, MTP_V, MTP_O, MTP_QN, MTP_KN, MTP_ROUTER,
 MTP_GATE_E, MTP_UP_E, MTP_DOWN_E, MTP_SH_GATE_INP, MTP_SH_GATE, MTP_SH_UP, MTP_SH_DOWN, MTP_HEAD, MTP_SLOTS) = range(31)


def mtp_specs(c: Config, n_exp, ff, lr=None):
    """[(slot, kind, ty, rows, cols)] of the drafter's tensors except the head (rows of the main output matrix)."""
    w = c.hc * c.d; lr = lr or c.hc_lr; sf = c.ff_sh or ff
    out = [(MTP_PRE_E, "vec:norm1", synth.F32, 1, c.d), (MTP_PRE_H, "vec:norm1", synth.F32, 1, w),
           (MTP_FC_E, "q", c.qtype, c.d, c.d), (MTP_FC_H, "q", c.qtype, c.d, c.d)]
    for base, inj in ((MTP_HCA_NORM, True), (MTP_HCF_NORM, True)):
        out += [(base, "vec:norm1", synth.F32, 1, w), (base + 1, "hc", c.hc_type, lr, w), (base + 2, "hc", c.hc_type, c.hc, w), (base + 3, "hc", c.hc_type, w, lr)]
    out += [(MTP_MIX_NORM, "vec:norm1", synth.F32, 1, w), (MTP_MIX_DOWN, "hc", c.hc_type, lr, w), (MTP_MIX_UP, "hc", c.hc_type, w, lr)]
    out += [(MTP_Q, "q", c.qtype, c.n_head * 2 * c.hd, c.d), (MTP_K, "q", c.qtype, c.n_kv * c.hd, c.d), (MTP_V, "q", c.qtype, c.n_kv * c.hd, c.d),
            (MTP_O, "q", c.qtype, c.d, c.n_head * c.hd), (MTP_QN, "vec:norm1", synth.F32, 1, c.hd), (MTP_KN, "vec:norm1", synth.F32, 1, c.hd),
            (MTP_ROUTER, "router", c.router_type, n_exp, c.d), (MTP_GATE_E, "q", c.qtype, n_exp * ff, c.d), (MTP_UP_E, "q", c.qtype, n_exp * ff, c.d),
            (MTP_DOWN_E, "q", c.qtype, n_exp * c.d, ff), (MTP_SH_GATE_INP, "vec:small", synth.F32, 1, c.d), (MTP_SH_GATE, "q", c.qtype, sf, c.d),
            (MTP_SH_UP, "q", c.qtype, sf, c.d), (MTP_SH_DOWN, "q", c.qtype, c.d, sf)]
    return out


def build_mtp_host(c: Config, hw: HostWeights, n_exp, ff, draft_ids, seed=7, lr=None):
    """dict slot -> (ty, rows, cols, bytes): synthetic drafter tensors, and as head the rows `draft_ids` of the main
    model's output matrix in its own type (the reference re-quantizes those rows to int8, mtp.rs:107)."""
    out = {}
    for slot, kind, ty, rows, cols in mtp_specs(c, n_exp, ff, lr):
        il, sl = (0, HCA_DOWN) if kind == "hc" else (0, ATTN_Q)          # scale range of a hyper-connection matrix or of a projection
        k2 = "q" if kind == "hc" else kind
        s = tensor_seed(seed, 99, slot)
        if k2 == "q" and ty not in (synth.F32, synth.F16, synth.BF16):
            b = synth.matrix(ty, rows, cols, s, *scale_range(c, il, sl, ty))
        else:
            b = host_tensor(c, seed, 99, slot, k2, ty, rows, cols)
        out[slot] = (ty, rows, cols, b)
    ty, rows, cols, b = hw.globals_[G_OUT]
    el, bs, _ = synth.GEOM[ty] if ty in synth.GEOM else (1, {synth.F32: 4, synth.F16: 2, synth.BF16: 2}[ty], None)
    rb = cols // el * bs
    ids = np.asarray(draft_ids, dtype=np.int64)
    out[MTP_HEAD] = (ty, ids.size, cols, np.ascontiguousarray(b.reshape(rows, rb)[ids]).reshape(-1))
    return out


def build_mtp_device(ctx, c: Config, n_exp, ff, n_draft, seed=7, lr=None):
    """The drafter's tensors with every quantized matrix generated on the device (benchmark sizes).  The head is a
    synthetic [n_draft][d] matrix of the main output matrix's type, not rows of that matrix: same shape and cost.
    Returns (tensors, raw_device_buffers)."""
    out, raw = {}, []
    specs = mtp_specs(c, n_exp, ff, lr) + [(MTP_HEAD, "q", c.qtype, n_draft, c.d)]
    for slot, kind, ty, rows, cols in specs:
        il, sl = (0, HCA_DOWN) if kind == "hc" else (0, ATTN_Q)
        k2 = "q" if kind == "hc" else kind
        if k2 == "q" and ty not in (synth.F32, synth.F16, synth.BF16):
            el, bs, _ = synth.GEOM[ty]
            nb = rows * (cols // el)
            dev = ctx.alloc(nb * bs)
            lo, hi = scale_range(c, il, sl, ty)
            ctx.synth_blocks(ty, nb, tensor_seed(seed, 99, slot), lo, hi, dev_out=dev)
            raw.append(dev)
            out[slot] = (ty, rows, cols, dev)
        else:
            out[slot] = (ty, rows, cols, host_tensor(c, seed, 99, slot, k2, ty, rows, cols))
    return out, raw
