"""Independent numpy statements used to pin the C++ oracle (and, through it, the HIP library).

Nothing here shares code with oracle/pyre_oracle.cpp: the codebooks are re-expanded from the header text,
the dequantizers are vectorised over blocks, and the block-level math (DeltaNet, attention, MoE, hyper-connections,
token step) is written in float64 from the format / architecture definitions.
"""
import hashlib
import os
import re

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# sha256 of the expanded little-endian tables, computed from the reference's iq_tables.rs by oracle/make_codebooks.py
IQ3S_SHA256 = "bd1af4945a1717c65610b0284e4628b9a1ba3b306fae3a06f6e5f597356e349f"
IQ2XS_SHA256 = "06e47aaca60b4dc1d9b5a3f34540437058a6b142b4d7a59d5ded769b4d1bf1de"
KSIGNS_SHA256 = "a76742a603f8beca5212ecce0f1f02f11a4887fd2f7c8b15aca0ea3eb3380c31"
IQ2XXS_SHA256 = "05826b5d3e472a3a78f196be62ac78acf81df0f909626e12ab9fa2a5d490dd54"
IQ1S_SHA256 = "07540ffc1aeaf6ad4d97e96b0fcc765aae39671d4ae4a27bbd0e796fde167c6a"      # IQ1S_GRID (iq_tables.rs:321 of the reference), 2048 x 8 int8
IQ2S_SHA256 = "e1aa1473412b0552c2174c30ef22ab4073f6a181b85a17056e8249bd2932fd88"
IQ3XXS_SHA256 = "46e35f5a997efdee6c99ce57854c8a0d4f0ff8ca57e5e8a60c0793ea580acf5d"
# the IQ4_NL / IQ4_XS non-linear levels (ggml's kvalues_iq4nl, iq_tables.rs:579 of the reference)
IQ4NL_VALUES = (-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113)


def _codes(path, name):
    txt = open(path).read()
    m = re.search(r"%s\[(\d+)\] = \{(.*?)\};" % name, txt, re.S)
    v = np.array([int(s) for s in re.findall(r"\d+", m.group(2))], dtype=np.uint32)
    assert v.size == int(m.group(1))
    return v


def codebooks(header=None):
    """(iq3s_grid u8[512,4], iq2xs_grid u8[512,8], ksigns u8[128]) expanded from a codebook header."""
    header = header or os.path.join(_ROOT, "oracle", "iq_codebooks.h")
    c3 = _codes(header, "kIq3sCode")
    c2 = _codes(header, "kIq2xsCode")
    g3 = np.stack([2 * ((c3 >> (3 * j)) & 7) + 1 for j in range(4)], axis=1).astype(np.uint8)
    tri = np.array([8, 25, 43], dtype=np.uint8)
    g2 = np.stack([tri[(c2 >> (2 * j)) & 3] for j in range(8)], axis=1).astype(np.uint8)
    i = np.arange(128, dtype=np.uint32)
    par = np.zeros(128, dtype=np.uint32)
    for b in range(7):
        par ^= (i >> b) & 1
    ks = (i | (par << 7)).astype(np.uint8)
    return g3, g2, ks


def codebooks_more(header=None):
    """(iq2xxs_grid u8[256,8], iq2s_grid u8[1024,8], iq3xxs_grid u8[256,4], iq4nl i8[16]) expanded from a codebook header."""
    header = header or os.path.join(_ROOT, "oracle", "iq_codebooks.h")
    tri = np.array([8, 25, 43], dtype=np.uint8)
    lv3 = np.array([4, 12, 20, 28, 36, 44, 52, 62], dtype=np.uint8)
    cxx, cs, c3 = _codes(header, "kIq2xxsCode"), _codes(header, "kIq2sCode"), _codes(header, "kIq3xxsCode")
    gxx = np.stack([tri[(cxx >> (2 * j)) & 3] for j in range(8)], axis=1).astype(np.uint8)
    gs = np.stack([tri[(cs >> (2 * j)) & 3] for j in range(8)], axis=1).astype(np.uint8)
    g3 = np.stack([lv3[(c3 >> (3 * j)) & 7] for j in range(4)], axis=1).astype(np.uint8)
    m = re.search(r"kIq4nlValues\[16\] = \{(.*?)\};", open(header).read(), re.S)
    kv = np.array([int(v) for v in re.findall(r"-?\d+", m.group(1))], dtype=np.int8)
    return gxx, gs, g3, kv


def codebook_iq1s(header=None):
    """iq1s_grid i8[2048, 8] expanded from a codebook header: byte j of entry e = ((code >> 2j) & 3) - 1."""
    header = header or os.path.join(_ROOT, "oracle", "iq_codebooks.h")
    c = _codes(header, "kIq1sCode")
    return np.stack([((c >> (2 * j)) & 3).astype(np.int8) - 1 for j in range(8)], axis=1).astype(np.int8)


def codebook_digests_more(header=None):
    gxx, gs, g3, kv = codebooks_more(header)
    return (hashlib.sha256(gxx.tobytes()).hexdigest(), hashlib.sha256(gs.tobytes()).hexdigest(), hashlib.sha256(g3.tobytes()).hexdigest(), tuple(int(v) for v in kv))


def codebook_digests(header=None):
    g3, g2, ks = codebooks(header)
    return (hashlib.sha256(g3.tobytes()).hexdigest(), hashlib.sha256(g2.tobytes()).hexdigest(), hashlib.sha256(ks.tobytes()).hexdigest())


def f16_to_f32(b):
    return np.ascontiguousarray(b).view(np.float16).astype(np.float32)


def _signs(s):
    """sign byte array [...] -> [..., 8] of +-1 float32 (bit j set = negative)."""
    return np.where((s[..., None] >> np.arange(8, dtype=np.uint8)) & 1, np.float32(-1), np.float32(1)).astype(np.float32)


def dequant(ty, raw, n):
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    g3, g2, ks = codebooks()
    if ty == 0:
        return raw[:4 * n].view(np.float32).copy()
    if ty == 1:
        return f16_to_f32(raw[:2 * n])
    if ty == 30:
        return (raw[:2 * n].view(np.uint16).astype(np.uint32) << 16).view(np.float32)
    if ty == 8:
        b = raw[:n // 32 * 34].reshape(-1, 34)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        return (b[:, 2:].view(np.int8).astype(np.float32) * d).reshape(-1)
    if ty == 12:
        b = raw[:n // 256 * 144].reshape(-1, 144)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1)
        mn = f16_to_f32(b[:, 2:4].copy()).reshape(-1)
        sc = b[:, 4:16].astype(np.uint32)
        s = np.empty((b.shape[0], 8), dtype=np.uint32); m = np.empty_like(s)
        for j in range(8):
            if j < 4:
                s[:, j] = sc[:, j] & 63; m[:, j] = sc[:, j + 4] & 63
            else:
                s[:, j] = (sc[:, j + 4] & 0xF) | ((sc[:, j - 4] >> 6) << 4)
                m[:, j] = (sc[:, j + 4] >> 4) | ((sc[:, j] >> 6) << 4)
        q = b[:, 16:].reshape(-1, 4, 32)
        out = np.empty((b.shape[0], 4, 2, 32), dtype=np.float32)
        for g in range(4):
            d1 = (d * s[:, 2 * g].astype(np.float32)).astype(np.float32)[:, None]
            m1 = (mn * m[:, 2 * g].astype(np.float32)).astype(np.float32)[:, None]
            d2 = (d * s[:, 2 * g + 1].astype(np.float32)).astype(np.float32)[:, None]
            m2 = (mn * m[:, 2 * g + 1].astype(np.float32)).astype(np.float32)[:, None]
            out[:, g, 0] = (d1 * (q[:, g] & 0xF).astype(np.float32)).astype(np.float32) - m1
            out[:, g, 1] = (d2 * (q[:, g] >> 4).astype(np.float32)).astype(np.float32) - m2
        return out.reshape(-1)
    if ty == 17:
        b = raw[:n // 256 * 74].reshape(-1, 74)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        qs = b[:, 2:66].copy().view(np.uint16).reshape(-1, 8, 4).astype(np.uint32)
        sc = b[:, 66:74]
        lo = ((d * (np.float32(0.5) + (sc & 0xF).astype(np.float32))).astype(np.float32) * np.float32(0.25)).astype(np.float32)
        hi = ((d * (np.float32(0.5) + (sc >> 4).astype(np.float32))).astype(np.float32) * np.float32(0.25)).astype(np.float32)
        db = np.stack([lo, lo, hi, hi], axis=2)                       # [nb, 8, 4]
        grid = g2[qs & 511].astype(np.float32)                        # [nb, 8, 4, 8]
        sg = _signs(ks[qs >> 9])
        return ((db[..., None] * grid).astype(np.float32) * sg).astype(np.float32).reshape(-1)
    if ty == 21:
        b = raw[:n // 256 * 110].reshape(-1, 110)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        qs = b[:, 2:66].reshape(-1, 8, 8).astype(np.uint32)           # [nb, sub-block, 8 index bytes]
        qh = b[:, 66:74].astype(np.uint32)                            # one byte per sub-block
        sg = b[:, 74:106].reshape(-1, 8, 4)
        sc = b[:, 106:110]
        nib = np.stack([sc & 0xF, sc >> 4], axis=2).reshape(-1, 8).astype(np.float32)
        db = (d * (np.float32(1) + np.float32(2) * nib)).astype(np.float32)   # d * (1 + 2 nib) -- integer valued, exact
        hbit = (qh[:, :, None] >> np.arange(8, dtype=np.uint32)) & 1   # bit k of qh goes with index byte k
        idx = qs | (hbit << 8)
        grid = g3[idx].astype(np.float32).reshape(-1, 8, 4, 8)         # two 4-byte entries per group of 8 values
        s = _signs(sg)
        return ((db[:, :, None, None] * grid).astype(np.float32) * s).astype(np.float32).reshape(-1)
    f = np.float32
    if ty == 2:                                                        # Q4_0: (nibble - 8) * d; low nibbles first, then high
        b = raw[:n // 32 * 18].reshape(-1, 18)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        q = np.concatenate([b[:, 2:] & 0xF, b[:, 2:] >> 4], axis=1).astype(np.int32) - 8
        return (q.astype(f) * d).astype(f).reshape(-1)
    if ty == 6:                                                        # Q5_0: fifth bit of element e is bit e of the u32 at byte 2
        b = raw[:n // 32 * 22].reshape(-1, 22)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        qh = b[:, 2:6].copy().view(np.uint32).reshape(-1, 1)
        hb = ((qh >> np.arange(32, dtype=np.uint32)) & 1).astype(np.int32)
        q = np.concatenate([b[:, 6:] & 0xF, b[:, 6:] >> 4], axis=1).astype(np.int32) + 16 * hb - 16
        return (q.astype(f) * d).astype(f).reshape(-1)
    if ty == 29:                                                       # IQ1_M: qs[32] | qh[16] | four u16 scale words whose top nibbles spell the f16 d
        b = raw[:n // 256 * 56].reshape(-1, 56)
        nb = b.shape[0]
        g1 = codebook_iq1s().astype(f)                                 # [2048, 8]
        sc = b[:, 48:56].copy().view(np.uint16).reshape(nb, 4).astype(np.uint32)
        su = ((sc[:, 0] >> 12) | ((sc[:, 1] >> 8) & 0xF0) | ((sc[:, 2] >> 4) & 0xF00) | (sc[:, 3] & 0xF000)).astype(np.uint16)
        d = su.view(np.float16).astype(f).reshape(nb, 1)
        qs = b[:, 0:32].reshape(nb, 8, 4).astype(np.uint32); qh = b[:, 32:48].reshape(nb, 8, 2).astype(np.uint32)
        ib = np.arange(8)
        w = sc[:, ib // 2]                                             # [nb, 8]: the scale word of sub-block ib
        s3a = (w >> (6 * (ib % 2))) & 7; s3b = (w >> (6 * (ib % 2) + 3)) & 7
        dl1 = (d * (2 * s3a + 1).astype(f)).astype(f); dl2 = (d * (2 * s3b + 1).astype(f)).astype(f)      # [nb, 8]
        hi = np.stack([(qh[:, :, 0] << 8) & 0x700, (qh[:, :, 0] << 4) & 0x700, (qh[:, :, 1] << 8) & 0x700, (qh[:, :, 1] << 4) & 0x700], axis=2)
        idx = qs | hi                                                  # [nb, 8, 4]
        neg = np.stack([qh[:, :, 0] & 0x08, qh[:, :, 0] & 0x80, qh[:, :, 1] & 0x08, qh[:, :, 1] & 0x80], axis=2) != 0
        delta = np.where(neg, f(-0.125), f(0.125)).astype(f)           # [nb, 8, 4]
        s = np.stack([dl1, dl1, dl2, dl2], axis=2)                     # groups 0, 1 of a sub-block use the first 3-bit scale, 2, 3 the second
        return (s[:, :, :, None] * (g1[idx] + delta[:, :, :, None]).astype(f)).astype(f).reshape(-1)
    if ty == 13:                                                       # Q5_K: d | dmin | scales[12] | qh[32] | ql[128]; (d*s) * (nibble + 16*bit) - dmin*m
        b = raw[:n // 256 * 176].reshape(-1, 176)
        nb = b.shape[0]
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1); mn = f16_to_f32(b[:, 2:4].copy()).reshape(-1)
        sc = b[:, 4:16].astype(np.uint32)
        s = np.empty((nb, 8), dtype=np.uint32); m = np.empty_like(s)
        for j in range(8):
            if j < 4:
                s[:, j] = sc[:, j] & 63; m[:, j] = sc[:, j + 4] & 63
            else:
                s[:, j] = (sc[:, j + 4] & 0xF) | ((sc[:, j - 4] >> 6) << 4)
                m[:, j] = (sc[:, j + 4] >> 4) | ((sc[:, j] >> 6) << 4)
        qh = b[:, 16:48].astype(np.int32); ql = b[:, 48:].reshape(nb, 4, 32).astype(np.int32)
        out = np.empty((nb, 8, 32), dtype=f)                               # sub-block 2j: low nibbles, 2j+1: high nibbles of the same 32 bytes
        for sb in range(8):
            nib = (ql[:, sb // 2] & 0xF) if sb % 2 == 0 else (ql[:, sb // 2] >> 4)
            q = (nib + 16 * ((qh >> sb) & 1)).astype(f)
            d1 = (d * s[:, sb].astype(f)).astype(f).reshape(nb, 1); m1 = (mn * m[:, sb].astype(f)).astype(f).reshape(nb, 1)
            out[:, sb] = ((d1 * q).astype(f) - m1).astype(f)
        return out.reshape(-1)
    if ty == 42:                                                       # Q2_0: 64 values per block, four 2-bit codes per byte (low bits first), (code - 1) * d
        b = raw[:n // 64 * 18].reshape(-1, 18)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        q = ((b[:, 2:, None].astype(np.int32) >> (2 * np.arange(4))) & 3).reshape(-1, 64) - 1
        return (q.astype(f) * d).astype(f).reshape(-1)
    if ty == 11:                                                       # Q3_K: hmask[32] | qs[64] | scales[12] | d; value = d*(sc6 - 32) * (low2 - (hbit ? 0 : 4))
        b = raw[:n // 256 * 110].reshape(-1, 110)
        nb = b.shape[0]
        hm = b[:, 0:32].astype(np.int32); qs = b[:, 32:96].reshape(nb, 2, 32).astype(np.int32); s12 = b[:, 96:108].astype(np.int32)
        d = f16_to_f32(b[:, 108:110].copy()).reshape(nb, 1)
        # sixteen 6-bit scales: low 4 bits from bytes 0..7 (low nibbles -> scales 0..7, high nibbles -> 8..15), high 2 bits from bytes 8..11
        lo4 = np.concatenate([s12[:, 0:8] & 0xF, s12[:, 0:8] >> 4], axis=1)                                  # [nb, 16]
        hi2 = np.stack([(s12[:, 8 + (k % 4)] >> (2 * (k // 4))) & 3 for k in range(16)], axis=1)             # scale k: byte 8 + k%4, bits 2*(k/4)
        sc6 = (lo4 | (hi2 << 4)) - 32
        dl = (d * sc6.astype(f)).astype(f)                                                                   # [nb, 16]: scale of values 16k .. 16k+15
        out = np.empty((nb, 2, 4, 32), dtype=np.int32)                                                       # [half of 128][shift step j][byte o]
        for nn in range(2):
            for j in range(4):
                hb = (hm >> (4 * nn + j)) & 1
                out[:, nn, j] = ((qs[:, nn] >> (2 * j)) & 3) - 4 * (1 - hb)
        q = out.reshape(nb, 16, 16).astype(f)                                                                # value index = nn*128 + j*32 + o; 16 per scale
        return (dl[:, :, None] * q).astype(f).reshape(-1)
    gxx, gs, g3x, kv = codebooks_more()
    kvf = kv.astype(f)
    if ty == 20:                                                       # IQ4_NL: d * level[nibble]
        b = raw[:n // 32 * 18].reshape(-1, 18)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        q = np.concatenate([b[:, 2:] & 0xF, b[:, 2:] >> 4], axis=1)
        return (d * kvf[q]).astype(f).reshape(-1)
    if ty == 23:                                                       # IQ4_XS: 6-bit sub-block scale = 4 low bits (byte 4..7) | 2 high bits (u16 at 2)
        b = raw[:n // 256 * 136].reshape(-1, 136)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        sh = b[:, 2:4].copy().view(np.uint16).astype(np.int32).reshape(-1, 1)
        ib = np.arange(8)
        lo4 = (b[:, 4:8][:, ib // 2].astype(np.int32) >> (4 * (ib % 2))) & 0xF
        ls = lo4 | (((sh >> (2 * ib)) & 3) << 4)
        dl = (d * (ls - 32).astype(f)).astype(f)                      # [nb, 8]
        qs = b[:, 8:].reshape(-1, 8, 16)
        q = np.concatenate([qs & 0xF, qs >> 4], axis=2)               # [nb, 8, 32]
        return (kvf[q] * dl[:, :, None]).astype(f).reshape(-1)
    if ty == 14:                                                       # Q6_K: (d * scale_i8) * (6-bit value - 32), 16 values per scale
        b = raw[:n // 256 * 210].reshape(-1, 210)
        nb = b.shape[0]
        ql = b[:, 0:128].reshape(nb, 2, 2, 32).astype(np.int32)        # [half][which 32 bytes][l]
        qh = b[:, 128:192].reshape(nb, 2, 32).astype(np.int32)
        sc = b[:, 192:208].copy().view(np.int8).reshape(nb, 2, 4, 2).astype(f)   # [half][quarter][l // 16]
        d = f16_to_f32(b[:, 208:210].copy()).reshape(nb, 1, 1, 1)
        q = np.empty((nb, 2, 4, 32), dtype=np.int32)
        for qd in range(4):
            nib = (ql[:, :, qd & 1] & 0xF) if qd < 2 else (ql[:, :, qd & 1] >> 4)
            q[:, :, qd] = (nib | (((qh >> (2 * qd)) & 3) << 4)) - 32
        scale = (d * sc).astype(f)                                     # [nb, 2, 4, 2]
        scale = np.repeat(scale, 16, axis=3)                           # per element l of the quarter
        return (scale * q.astype(f)).astype(f).reshape(-1)
    g3, g2, ks = codebooks()
    if ty == 16:                                                       # IQ2_XXS: 8 bytes per 32 values: 4 grid indices, then 4x7 sign bits + 4 scale bits
        b = raw[:n // 256 * 66].reshape(-1, 66)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        qs = b[:, 2:66].reshape(-1, 8, 8)
        a1 = qs[:, :, 4:8].copy().view(np.uint32).reshape(-1, 8)
        db = ((d * (f(0.5) + (a1 >> 28).astype(f))).astype(f) * f(0.25)).astype(f)
        grid = gxx[qs[:, :, 0:4]].astype(f)                             # [nb, 8, 4, 8]
        sg = _signs(ks[(a1[:, :, None] >> (7 * np.arange(4, dtype=np.uint32))) & 127])
        return ((db[:, :, None, None] * grid).astype(f) * sg).astype(f).reshape(-1)
    if ty == 22:                                                       # IQ2_S: 10-bit grid index = byte | 2 bits of qh; one scale nibble per 16 values
        b = raw[:n // 256 * 82].reshape(-1, 82)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        qs = b[:, 2:34].reshape(-1, 8, 4).astype(np.uint32)
        sg = b[:, 34:66].reshape(-1, 8, 4)
        qh = b[:, 66:74].astype(np.uint32)
        sc = b[:, 74:82]
        hi2 = (qh[:, :, None] >> (2 * np.arange(4, dtype=np.uint32))) & 3
        grid = gs[qs | (hi2 << 8)].astype(f)                            # [nb, 8, 4, 8]
        lo = ((d * (f(0.5) + (sc & 0xF).astype(f))).astype(f) * f(0.25)).astype(f)
        hi = ((d * (f(0.5) + (sc >> 4).astype(f))).astype(f) * f(0.25)).astype(f)
        db = np.stack([lo, lo, hi, hi], axis=2)
        return ((db[..., None] * grid).astype(f) * _signs(sg)).astype(f).reshape(-1)
    if ty == 18:                                                       # IQ3_XXS: 64 grid indices (4 values each), then per 32 values a u32 of 4x7 sign bits + 4 scale bits
        b = raw[:n // 256 * 98].reshape(-1, 98)
        d = f16_to_f32(b[:, 0:2].copy()).reshape(-1, 1)
        qs = b[:, 2:66].reshape(-1, 8, 4, 2)
        a = b[:, 66:98].copy().view(np.uint32).reshape(-1, 8)
        db = ((d * (f(0.5) + (a >> 28).astype(f))).astype(f) * f(0.5)).astype(f)
        grid = g3x[qs].astype(f).reshape(-1, 8, 4, 8)
        sg = _signs(ks[(a[:, :, None] >> (7 * np.arange(4, dtype=np.uint32))) & 127])
        return ((db[:, :, None, None] * grid).astype(f) * sg).astype(f).reshape(-1)
    raise ValueError(ty)


# ---- hand packers for known-answer blocks -----------------------------------------------------------------------
def f16_bytes(v):
    return np.array([v], dtype=np.float16).view(np.uint8)


def pack_iq3s(d, qs, qh, signs, scales):
    b = np.zeros(110, dtype=np.uint8)
    b[0:2] = f16_bytes(d); b[2:66] = qs; b[66:74] = qh; b[74:106] = signs; b[106:110] = scales
    return b


def pack_iq2xs(d, qs16, scales):
    b = np.zeros(74, dtype=np.uint8)
    b[0:2] = f16_bytes(d); b[2:66] = np.asarray(qs16, dtype=np.uint16).view(np.uint8); b[66:74] = scales
    return b


def pack_q4k(d, dmin, s, m, q):
    """s, m: 8 six-bit scale / min values; q: 256 four-bit values in element order."""
    b = np.zeros(144, dtype=np.uint8)
    b[0:2] = f16_bytes(d); b[2:4] = f16_bytes(dmin)
    s = np.asarray(s, dtype=np.uint8); m = np.asarray(m, dtype=np.uint8)
    sc = np.zeros(12, dtype=np.uint8)
    for j in range(4):
        sc[j] = (s[j] & 63) | ((s[j + 4] >> 4) << 6)
        sc[j + 4] = (m[j] & 63) | ((m[j + 4] >> 4) << 6)
        sc[j + 8] = (s[j + 4] & 0xF) | ((m[j + 4] & 0xF) << 4)
    b[4:16] = sc
    q = np.asarray(q, dtype=np.uint8).reshape(4, 2, 32)
    b[16:] = (q[:, 0] | (q[:, 1] << 4)).reshape(-1)
    return b


def pack_q8_0(d, q):
    b = np.zeros(34, dtype=np.uint8)
    b[0:2] = f16_bytes(d); b[2:] = np.asarray(q, dtype=np.int8).view(np.uint8)
    return b


# ---- float64 block math -----------------------------------------------------------------------------------------
def sigm(x):
    return 1.0 / (1.0 + np.exp(-x))


def silu(x):
    return x * sigm(x)


def softplus(x):
    return np.where(x > 20.0, x, np.log1p(np.exp(np.minimum(x, 20.0))))


def rms(x, w, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def kv4_roundtrip(x):
    x = np.asarray(x, dtype=np.float32).reshape(-1, 32)
    m = np.abs(x).max(axis=1, keepdims=True)
    s = np.where((m > 0) & np.isfinite(m), (m / np.float32(7)).astype(np.float32), np.float32(0))
    with np.errstate(divide="ignore", invalid="ignore"):
        r = (x / s).astype(np.float32)
    q = np.where(s > 0, np.clip(np.sign(r) * np.floor(np.abs(r) + np.float32(0.5)), -7, 7), 0).astype(np.int32).astype(np.float32)  # integer code: no -0
    return (q * s).astype(np.float32).reshape(-1), q.astype(np.int32).reshape(-1), s.reshape(-1)


def gdn_step(nk, nv, dk, dv, conv_k, eps, a, dt, conv_w, norm_w, qkv, z, beta, alpha, conv_state, S):
    """One token, float64.  conv_state [(k-1), ch] oldest first, S [nv, dk, dv]. Returns (out, conv_state', S')."""
    ch = 2 * nk * dk + nv * dv
    conv_w = np.asarray(conv_w, dtype=np.float64).reshape(ch, conv_k)
    win = np.concatenate([np.asarray(conv_state, dtype=np.float64).reshape(conv_k - 1, ch), np.asarray(qkv, dtype=np.float64)[None]], axis=0)
    co = silu((win * conv_w.T).sum(axis=0))
    q = co[:nk * dk].reshape(nk, dk); k = co[nk * dk:2 * nk * dk].reshape(nk, dk); v = co[2 * nk * dk:].reshape(nv, dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) / np.sqrt(dk)
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    S = np.asarray(S, dtype=np.float64).reshape(nv, dk, dv).copy()
    out = np.empty((nv, dv))
    for h in range(nv):
        kh = h % nk
        g = np.exp(softplus(float(alpha[h]) + float(dt[h])) * float(a[h])); b = sigm(float(beta[h]))
        S[h] *= g
        mem = S[h].T @ k[kh]
        delta = (v[h] - mem) * b
        S[h] += np.outer(k[kh], delta)
        o = S[h].T @ q[kh]
        out[h] = rms(o, np.asarray(norm_w, dtype=np.float64), eps) * sigm(np.asarray(z, dtype=np.float64)[h * dv:(h + 1) * dv])
    return out.reshape(-1), win[1:], S


def rope(v, pos, n_rot, inv, mscale=1.0):
    v = np.array(v, dtype=np.float64); half = n_rot // 2
    ang = (np.float32(pos) * np.asarray(inv, dtype=np.float32)).astype(np.float64)   # the angle itself is an f32 product (qwen4exp_gguf.rs:530)
    c, s = np.cos(ang) * mscale, np.sin(ang) * mscale
    x0, x1 = v[..., :half].copy(), v[..., half:n_rot].copy()
    v[..., :half] = x0 * c - x1 * s
    v[..., half:n_rot] = x1 * c + x0 * s
    return v


def yarn_inv(n_rot, base, ctx_train, ctx):
    """float64 statement of the YaRN frequency table (llama.cpp / transformers defaults: beta_fast 32, beta_slow 1):
    (inverse frequencies, magnitude factor)."""
    i = np.arange(n_rot // 2, dtype=np.float64)
    plain = np.float64(np.float32(base)) ** (-2.0 * i / n_rot)
    if not (ctx_train > 0 and ctx > ctx_train):
        return plain, 1.0
    scale = ctx / ctx_train
    corr = lambda rot: n_rot * np.log(ctx_train / (rot * 2 * np.pi)) / (2 * np.log(base))
    low = max(np.floor(corr(32.0)), 0.0); high = min(np.ceil(corr(1.0)), n_rot // 2 - 1)
    ramp = np.ones_like(i) if abs(high - low) < 1e-6 else np.clip((i - low) / (high - low), 0.0, 1.0)
    return plain / scale * (1 - ramp) + plain * ramp, 1.0 + 0.1 * np.log(scale)


def qsa_select(iq, ib, n, ratio, budget):
    """Positions a query with n visible tokens attends to (ascending), or None while dense.  iq [nh][ihd] normalised and
    rotated index queries, ib [n // ratio][ihd] pooled block keys (float64).  Blocks ordered by (score desc, index asc)."""
    if n <= budget + ratio - 1:
        return None
    nb = n // ratio
    sc = np.maximum(ib[:nb] @ iq.T, 0.0).sum(1) / np.sqrt(iq.shape[1])
    order = sorted(range(nb), key=lambda b: (-sc[b], b))[:budget // ratio]
    pos = [p for b in sorted(order) for p in range(b * ratio, (b + 1) * ratio)] + list(range(nb * ratio, n))
    return np.array(pos, dtype=np.int64)


def qsa_pool(ik_rows, ikn, eps, first_pos, n_rot, inv, mscale=1.0):
    """Block key: mean of the block's raw index keys, RMSNorm, RoPE at the block's first position."""
    return rope(rms(np.asarray(ik_rows, dtype=np.float64).mean(0), np.asarray(ikn, dtype=np.float64), eps), first_pos, n_rot, inv, mscale)


def attn_step(nh, nkv, hd, n_rot, eps, inv, qn, kn, q, k, v, pos, K, V, packed_below=0, positions=None, mscale=1.0):
    """One token at position pos, float64. K,V [pos, nkv*hd] caches (f32 content). Returns (out, k_row, v_row).
    positions: the attended subset (ascending), default every visible position."""
    k = rope(rms(np.asarray(k, dtype=np.float64).reshape(nkv, hd), np.asarray(kn, dtype=np.float64), eps), pos, n_rot, inv, mscale)
    Kf = np.concatenate([np.asarray(K, dtype=np.float64).reshape(pos, nkv * hd), k.reshape(1, -1)], axis=0)
    Vf = np.concatenate([np.asarray(V, dtype=np.float64).reshape(pos, nkv * hd), np.asarray(v, dtype=np.float64).reshape(1, -1)], axis=0)
    Ke, Ve = Kf.copy(), Vf.copy()
    if packed_below:
        Ke[:packed_below] = kv4_roundtrip(Kf[:packed_below].astype(np.float32))[0].reshape(packed_below, -1)
        Ve[:packed_below] = kv4_roundtrip(Vf[:packed_below].astype(np.float32))[0].reshape(packed_below, -1)
    q = np.asarray(q, dtype=np.float64).reshape(nh, 2 * hd)
    out = np.empty((nh, hd)); grp = nh // nkv
    for h in range(nh):
        qh = rope(rms(q[h, :hd], np.asarray(qn, dtype=np.float64), eps), pos, n_rot, inv, mscale)
        kvh = h // grp
        Ks, Vs = (Ke, Ve) if positions is None else (Ke[positions], Ve[positions])
        sc = Ks[:, kvh * hd:(kvh + 1) * hd] @ qh / np.sqrt(hd)
        w = np.exp(sc - sc.max()); w /= w.sum()
        out[h] = (w[:, None] * Vs[:, kvh * hd:(kvh + 1) * hd]).sum(0) * sigm(q[h, hd:])
    return out.reshape(-1), Kf[-1].astype(np.float32), Vf[-1].astype(np.float32)


def top_k(r, k):
    r = np.asarray(r, dtype=np.float64).copy(); r[np.isnan(r)] = -np.inf
    order = sorted(range(r.size), key=lambda e: (-r[e], e))[:k]
    idx = np.array(sorted(order))
    mx = r[idx].max()
    if not np.isfinite(mx):
        return idx, np.full(k, 1.0 / k)
    w = np.exp(r[idx] - mx)
    return idx, w / w.sum()


def moe_ffn(d, n_exp, k, ff, W, x):
    """W: dict of dense float64 matrices router [E,d], gate_e [E,ff,d], up_e [E,ff,d], down_e [E,d,ff], sh_gate_inp [d],
    sh_gate [sf,d], sh_up [sf,d], sh_down [d,sf].  x [d]."""
    x = np.asarray(x, dtype=np.float64)
    lg = W["router"] @ x
    y = W["sh_down"] @ (silu(W["sh_gate"] @ x) * (W["sh_up"] @ x))
    y = y * sigm(W["sh_gate_inp"] @ x)
    idx, w = top_k(lg, k)
    for e, we in zip(idx, w):
        h = silu(W["gate_e"][e] @ x) * (W["up_e"][e] @ x)
        y = y + we * (W["down_e"][e] @ h)
    return y, idx, w


def hc_mix(d, hc, eps, norm, down, inject, up, x):
    x = np.asarray(x, dtype=np.float64).reshape(hc, d)
    xn = np.stack([rms(x[s], np.asarray(norm, dtype=np.float64)[s * d:(s + 1) * d], eps) for s in range(hc)]).reshape(-1)
    lo = silu((down @ xn) / hc)
    inj = (inject @ xn) / hc if inject is not None else np.zeros(hc)
    gate = up @ lo
    mixed = (xn * sigm(gate)).reshape(hc, d).sum(0) / hc
    return mixed, inj


def hc_combine(d, hc, x, out, inj):
    x = np.asarray(x, dtype=np.float64).reshape(hc, d).copy()
    for s in range(hc):
        x[s] += out * (2.0 * sigm(inj[s]))
    return x.reshape(-1)
