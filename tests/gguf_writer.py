"""Minimal GGUF v3 writer for the tests (layout per the container format the reference reads, gguf_q.rs:297-320):
magic, version, tensor count, kv count, key/values, tensor infos (name, dims, type, offset), padding to the alignment,
tensor data at aligned offsets."""
import struct

import numpy as np

from pyre_amd import modelgen as mg

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}


def _s(b):
    b = b.encode() if isinstance(b, str) else b
    return struct.pack("<Q", len(b)) + b


def _val(t, v):
    if t == STR:
        return _s(v)
    if t == ARR:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(_val(et, x) for x in items)
    return struct.pack(_FMT[t], v)


def write(path, meta, tensors, alignment=32, version=3, write_alignment_key=None):
    """meta: [(key, type, value)], tensors: [(name, shape (GGUF order: shape[0] = cols), ggml type, bytes)]."""
    if write_alignment_key is None:
        write_alignment_key = alignment != 32
    meta = list(meta)
    if write_alignment_key:
        meta.append(("general.alignment", U32, alignment))
    head = b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(meta))
    for k, t, v in meta:
        head += _s(k) + struct.pack("<I", t) + _val(t, v)
    off = 0; infos = b""; blobs = []
    for name, shape, ty, data in tensors:
        data = bytes(np.ascontiguousarray(data).tobytes()) if not isinstance(data, (bytes, bytearray)) else bytes(data)
        infos += _s(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape) + struct.pack("<IQ", ty, off)
        blobs.append((off, data))
        off = (off + len(data) + alignment - 1) // alignment * alignment
    head += infos
    pad = (-len(head)) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        base = f.tell()
        for o, data in blobs:
            f.seek(base + o); f.write(data)
        f.truncate(base + off)                       # zero padding up to the alignment after the last tensor


LAYER_NAMES = {
    mg.HCA_NORM: "hc_attn_norm.weight", mg.HCA_DOWN: "hc_attn_down.weight", mg.HCA_INJECT: "hc_attn_inject.weight", mg.HCA_UP: "hc_attn_up.weight",
    mg.HCF_NORM: "hc_ffn_norm.weight", mg.HCF_DOWN: "hc_ffn_down.weight", mg.HCF_INJECT: "hc_ffn_inject.weight", mg.HCF_UP: "hc_ffn_up.weight",
    mg.ATTN_Q: "attn_q.weight", mg.ATTN_K: "attn_k.weight", mg.ATTN_V: "attn_v.weight", mg.ATTN_O: "attn_output.weight", mg.ATTN_QN: "attn_q_norm.weight", mg.ATTN_KN: "attn_k_norm.weight",
    mg.LIN_QKV: "attn_qkv.weight", mg.LIN_Z: "attn_gate.weight", mg.LIN_BETA: "ssm_beta.weight", mg.LIN_ALPHA: "ssm_alpha.weight", mg.LIN_A: "ssm_a", mg.LIN_DT: "ssm_dt.bias",
    mg.LIN_CONV: "ssm_conv1d.weight", mg.LIN_NORM: "ssm_norm.weight", mg.LIN_OUT: "ssm_out.weight",
    mg.ROUTER: "ffn_gate_inp.weight", mg.GATE_E: "ffn_gate_exps.weight", mg.UP_E: "ffn_up_exps.weight", mg.DOWN_E: "ffn_down_exps.weight",
    mg.SH_GATE_INP: "ffn_gate_inp_shexp.weight", mg.SH_GATE: "ffn_gate_shexp.weight", mg.SH_UP: "ffn_up_shexp.weight", mg.SH_DOWN: "ffn_down_shexp.weight",
    mg.IDX_Q: "indexer.q_proj.weight", mg.IDX_K: "indexer.k_proj.weight", mg.IDX_QN: "indexer.q_norm.weight", mg.IDX_KN: "indexer.k_norm.weight",
    mg.PLE_KEY: "ple_key.weight", mg.PLE_VALUE: "ple_value.weight", mg.PLE_NK: "ple_norm_key.weight", mg.PLE_NQ: "ple_norm_query.weight", mg.PLE_NC: "ple_norm_conv.weight",
    mg.PLE_CONV: "ple_conv1d.weight",
}
GLOBAL_NAMES = {mg.G_EMBD: "token_embd.weight", mg.G_HEAD_NORM: "output_hc_norm.weight", mg.G_HEAD_DOWN: "output_hc_down.weight", mg.G_HEAD_UP: "output_hc_up.weight", mg.G_OUT: "output.weight", mg.G_PLE_TAB: "per_layer_token_embd.weight"}


def model_meta(c):
    a = "qwen4exp."
    return [("general.architecture", STR, "qwen4exp"), (a + "block_count", U32, c.n_layers), (a + "embedding_length", U32, c.d),
            (a + "hyper_connection.count", U32, c.hc), (a + "hyper_connection.low_rank", U32, c.hc_lr), (a + "attention.head_count", U32, c.n_head),
            (a + "attention.head_count_kv", U32, c.n_kv), (a + "attention.key_length", U32, c.hd), (a + "rope.dimension_count", U32, c.n_rot),
            (a + "rope.freq_base", F32, c.rope_base), (a + "attention.layer_norm_rms_epsilon", F32, c.eps), (a + "expert_count", U32, c.n_exp),
            (a + "expert_used_count", U32, c.top_k), (a + "expert_feed_forward_length", U32, c.ff_exp), (a + "ssm.group_count", U32, c.lin_nk),
            (a + "ssm.time_step_rank", U64, c.lin_nv), (a + "ssm.state_size", I32, c.lin_dk), (a + "ssm.conv_kernel", U16, c.conv_k),
            (a + "full_attention_interval", U8, c.full_every), (a + "context_length", U32, c.ctx_train or 262144), ("tokenizer.ggml.tokens", ARR, (STR, ["a", "b"]))] + \
           ([(a + "attention.indexer.head_count", U32, c.idx_nh), (a + "attention.indexer.key_length", U32, c.idx_hd), (a + "attention.indexer.top_k", U32, c.idx_budget),
             (a + "attention.compress_ratios", ARR, (U32, [1, c.idx_ratio, 2] if c.idx_ratio > 2 else [c.idx_ratio]))] if c.idx_nh > 0 else []) + \
           ([(a + "ple.layers", ARR, (U32, list(c.ple_layers))), (a + "ple.ngram_size", U32, c.ple_ngram), (a + "ple.heads_per_ngram", U32, c.ple_per_gram), (a + "ple.conv_kernel", U32, c.ple_conv_k),
             (a + "ple.eos_token_id", U32, c.ple_eos), (a + "embedding_length_per_layer_input", U32, c.ple_dim), (a + "ple.layer_multipliers", ARR, (U64, list(c.ple_mult))),
             (a + "ple.head_offsets", ARR, (U64, list(c.ple_off))), (a + "ple.head_vocab_sizes", ARR, (U64, list(c.ple_vocab)))] if c.ple_layers else [])


def model_tensors(c, hw):
    """The host weight set as GGUF tensors: 2-D [cols, rows]; expert stacks 3-D [cols, rows per expert, experts]."""
    out = []
    for il in range(c.n_layers):
        for slot, e in sorted(hw.layers[il].items()):
            if e is None:
                continue
            ty, rows, cols, data = e
            shape = [cols, rows // c.n_exp, c.n_exp] if slot in (mg.GATE_E, mg.UP_E, mg.DOWN_E) else ([cols] if rows == 1 else [cols, rows])
            out.append(("blk.%d.%s" % (il, LAYER_NAMES[slot]), shape, ty, data))
    for slot, e in sorted(hw.globals_.items()):
        ty, rows, cols, data = e
        out.append((GLOBAL_NAMES[slot], [cols] if rows == 1 else [cols, rows], ty, data))
    return out
