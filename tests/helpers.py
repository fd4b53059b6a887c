"""Shared test helpers: oracle tensors / models from pyre_amd.modelgen weight sets, dense float64 views."""
import numpy as np

import np_ref
import orc
from pyre_amd import modelgen as mg


def relerr(a, b):
    a = np.asarray(a, dtype=np.float64).reshape(-1); b = np.asarray(b, dtype=np.float64).reshape(-1)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def orc_tensor(entry):
    ty, rows, cols, b = entry
    return orc.tensor(ty, rows, cols, b)


def orc_cfg(c):
    from pyre_amd.lib import fill_cfg
    return fill_cfg(orc.Cfg(), c)


def orc_model(hw, threads=4):
    c = hw.cfg
    lt = []
    for il in range(c.n_layers):
        for slot in range(mg.LAYER_SLOTS):
            e = hw.layers[il].get(slot)
            lt.append(orc_tensor(e) if e is not None else orc.Tensor(0, 0, 0, None))
    g = [orc_tensor(hw.globals_[s]) if s in hw.globals_ else orc.Tensor(0, 0, 0, None) for s in range(mg.GLOBAL_SLOTS)]
    return orc.Model(orc_cfg(c), lt, g, threads=threads, keep=(hw,))


def dense(entry):
    ty, rows, cols, b = entry
    return np_ref.dequant(ty, b, rows * cols).reshape(rows, cols).astype(np.float64)


def np_forward_tokens(hw, ids):
    """float64 numpy statement of the token loop (one token at a time); returns logits after each token."""
    c = hw.cfg; d, hc = c.d, c.hc
    inv, ms = np_ref.yarn_inv(c.n_rot, c.rope_base, c.ctx_train, c.ctx)
    L = [{s: (dense(e) if e[0] != 0 or e[1] > 1 else e[3].view(np.float32).astype(np.float64)) for s, e in lay.items()} for lay in hw.layers]
    G = {s: (dense(e) if e[1] > 1 else e[3].view(np.float32).astype(np.float64)) for s, e in hw.globals_.items()}
    conv = {}; S = {}; K = {}; V = {}; IK = {}; IB = {}
    for il in range(c.n_layers):
        if c.full(il):
            K[il] = np.zeros((0, c.n_kv * c.hd), np.float32); V[il] = np.zeros((0, c.n_kv * c.hd), np.float32)
            IK[il] = np.zeros((0, c.idx_hd)); IB[il] = np.zeros((0, c.idx_hd))
        else:
            conv[il] = np.zeros((c.conv_k - 1, c.ch)); S[il] = np.zeros((c.lin_nv, c.lin_dk, c.lin_dv))
    out = []
    for pos, tok in enumerate(ids):
        x = np.tile(G[mg.G_EMBD][tok], hc)
        for il in range(c.n_layers):
            W = L[il]
            m, inj = np_ref.hc_mix(d, hc, c.eps, W[mg.HCA_NORM], W[mg.HCA_DOWN], W[mg.HCA_INJECT], W[mg.HCA_UP], x)
            if c.full(il):
                n = pos + 1
                pb = orc.packed_boundary(n, c.kv_bits, c.kv_recent)
                positions = None
                if c.idx_nh > 0 and mg.IDX_Q in W:
                    IK[il] = np.concatenate([IK[il], (W[mg.IDX_K] @ m)[None]])
                    if n % c.idx_ratio == 0:
                        b = n // c.idx_ratio - 1
                        IB[il] = np.concatenate([IB[il], np_ref.qsa_pool(IK[il][b * c.idx_ratio:n], W[mg.IDX_KN], c.eps, b * c.idx_ratio, c.n_rot, inv, ms)[None]])
                    iq = (W[mg.IDX_Q] @ m).reshape(c.idx_nh, c.idx_hd)
                    iq = np.stack([np_ref.rope(np_ref.rms(iq[h], W[mg.IDX_QN], c.eps), pos, c.n_rot, inv, ms) for h in range(c.idx_nh)])
                    positions = np_ref.qsa_select(iq, IB[il], n, c.idx_ratio, c.idx_budget)
                o, kr, vr = np_ref.attn_step(c.n_head, c.n_kv, c.hd, c.n_rot, c.eps, inv, W[mg.ATTN_QN], W[mg.ATTN_KN],
                                             W[mg.ATTN_Q] @ m, W[mg.ATTN_K] @ m, W[mg.ATTN_V] @ m, pos, K[il], V[il], pb, positions=positions, mscale=ms)
                K[il] = np.concatenate([K[il], kr[None]]); V[il] = np.concatenate([V[il], vr[None]])
                o = W[mg.ATTN_O] @ o
            else:
                o, conv[il], S[il] = np_ref.gdn_step(c.lin_nk, c.lin_nv, c.lin_dk, c.lin_dv, c.conv_k, c.eps, W[mg.LIN_A], W[mg.LIN_DT],
                                                     W[mg.LIN_CONV], W[mg.LIN_NORM], W[mg.LIN_QKV] @ m, W[mg.LIN_Z] @ m,
                                                     W[mg.LIN_BETA] @ m, W[mg.LIN_ALPHA] @ m, conv[il], S[il])
                o = W[mg.LIN_OUT] @ o
            x = np_ref.hc_combine(d, hc, x, o, inj)
            m, inj = np_ref.hc_mix(d, hc, c.eps, W[mg.HCF_NORM], W[mg.HCF_DOWN], W[mg.HCF_INJECT], W[mg.HCF_UP], x)
            sf = W[mg.SH_GATE].shape[0]
            Wm = {"router": W[mg.ROUTER], "gate_e": W[mg.GATE_E].reshape(c.n_exp, c.ff_exp, d), "up_e": W[mg.UP_E].reshape(c.n_exp, c.ff_exp, d),
                  "down_e": W[mg.DOWN_E].reshape(c.n_exp, d, c.ff_exp), "sh_gate_inp": W[mg.SH_GATE_INP], "sh_gate": W[mg.SH_GATE],
                  "sh_up": W[mg.SH_UP], "sh_down": W[mg.SH_DOWN]}
            o, _, _ = np_ref.moe_ffn(d, c.n_exp, c.top_k, c.ff_exp, Wm, m)
            x = np_ref.hc_combine(d, hc, x, o, inj)
        h, _ = np_ref.hc_mix(d, hc, c.eps, G[mg.G_HEAD_NORM], G[mg.G_HEAD_DOWN], None, G[mg.G_HEAD_UP], x)
        out.append(G[mg.G_OUT] @ h)
    return np.array(out)


def orc_mtp(om, mt, n_exp, top_k, ff, window, draft_ids):
    """The oracle's drafter over a modelgen.build_mtp_host tensor dict."""
    ts = [orc_tensor(mt[s]) if s in mt else orc.Tensor(0, 0, 0, None) for s in range(mg.MTP_SLOTS)]
    return orc.Mtp(om, n_exp, top_k, ff, window, ts, draft_ids, keep=(mt,))


def write_safetensors(path, tensors, meta=None, dtype="BF16"):
    """A safetensors file of 16-bit tensors given as uint16 arrays (name -> array), in dict order."""
    import json
    hdr = {}; off = 0; blobs = []
    if meta is not None:
        hdr["__metadata__"] = meta
    for name, arr in tensors.items():
        b = np.ascontiguousarray(arr, dtype=np.uint16).tobytes()
        hdr[name] = {"dtype": dtype, "shape": list(arr.shape), "data_offsets": [off, off + len(b)]}; off += len(b); blobs.append(b)
    h = json.dumps(hdr).encode(); h += b" " * (-len(h) % 8)
    with open(path, "wb") as f:
        f.write(len(h).to_bytes(8, "little")); f.write(h)
        for b in blobs:
            f.write(b)
