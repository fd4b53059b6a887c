"""Synthetic GGUF tensors for the benchmark configurations (host side, numpy).

The reference ships no quantizer, so "random-init weights quantized to IQ3_S" means what its own
micro-benchmarks do (qdot.rs:823-859, qn_cube.rs:7216-7249): random payload bytes with sane f16
scales.  The generator is counter based so that the HIP library can produce the same bytes on the
device (pyre_synth_blocks) for tensors too large to push through the host:

  word(S, i)   = mix64(S + (i + 1) * 0x9E3779B97F4A7C15)                      (splitmix64 finaliser)
  payload byte k of the tensor = byte (k % 8) of word(S, k // 8)              (little endian)
  scale word of block b        = word(S ^ 0xD1B54A32D192ED03, b)
  d     = f16( lo + (hi - lo) * ((w >> 40)          * 2^-24) )   round-to-nearest-even
  dmin  = f16( lo + (hi - lo) * (((w >> 16) & 0xFFFFFF) * 2^-24) )   (Q4_K only)
Every f16 scale field of a block is overwritten after the payload bytes are laid down.
"""
import numpy as np

GOLDEN = np.uint64(0x9E3779B97F4A7C15)
SCALE_SALT = np.uint64(0xD1B54A32D192ED03)

# ggml type id -> (elements per block, bytes per block, byte offsets of the f16 scale fields)
GEOM = {8: (32, 34, (0,)), 12: (256, 144, (0, 2)), 17: (256, 74, (0,)), 21: (256, 110, (0,)),
        0: (1, 4, ()), 1: (1, 2, ()), 30: (1, 2, ()),
        2: (32, 18, (0,)), 6: (32, 22, (0,)), 14: (256, 210, (208,)), 16: (256, 66, (0,)), 18: (256, 98, (0,)),
        20: (32, 18, (0,)), 22: (256, 82, (0,)), 23: (256, 136, (0,)), 11: (256, 110, (108,)), 42: (64, 18, (0,)), 13: (256, 176, (0, 2)),
        29: (256, 56, (-1,))}        # IQ1_M: the f16 scale is scattered over the top nibbles of the four scale words (bytes 49, 51, 53, 55)
Q8_0, Q4_K, IQ2_XS, IQ3_S, F32, F16, BF16 = 8, 12, 17, 21, 0, 1, 30
Q4_0, Q5_0, Q6_K, IQ2_XXS, IQ3_XXS, IQ4_NL, IQ2_S, IQ4_XS, Q3_K, Q2_0, Q5_K, IQ1_M = 2, 6, 14, 16, 18, 20, 22, 23, 11, 42, 13, 29


def mix64(z):
    z = z.astype(np.uint64, copy=True)
    z ^= z >> np.uint64(30); z *= np.uint64(0xBF58476D1CE4E5B9)
    z ^= z >> np.uint64(27); z *= np.uint64(0x94D049BB133111EB)
    z ^= z >> np.uint64(31)
    return z


def words(seed, n, start=0):
    with np.errstate(over="ignore"):
        i = np.arange(start + 1, start + n + 1, dtype=np.uint64)
        return mix64(np.uint64(seed) + i * GOLDEN)


def blocks(ty, n_blocks, seed, d_lo=1e-3, d_hi=2e-2):
    """n_blocks raw GGUF blocks of type `ty` as a uint8 array."""
    _, bs, fields = GEOM[ty]
    nbytes = n_blocks * bs
    raw = words(seed, (nbytes + 7) // 8).view(np.uint8)[:nbytes].copy()
    if fields:
        w = words(np.uint64(seed) ^ SCALE_SALT, n_blocks)
        lo, hi = np.float32(d_lo), np.float32(d_hi)
        b = raw.reshape(n_blocks, bs)
        for fi, off in enumerate(fields):
            bits = (w >> np.uint64(40)) if fi == 0 else ((w >> np.uint64(16)) & np.uint64(0xFFFFFF))
            u = bits.astype(np.float32) * np.float32(2.0 ** -24)
            v = (lo + (hi - lo) * u).astype(np.float32).astype(np.float16)
            if off < 0:
                h = v.view(np.uint16).astype(np.uint32)
                for k in range(4):
                    b[:, 49 + 2 * k] = (b[:, 49 + 2 * k] & 0x0F) | (((h >> (4 * k)) & 0xF) << 4).astype(np.uint8)
                continue
            b[:, off:off + 2] = v.view(np.uint8).reshape(n_blocks, 2)
    return raw


def matrix(ty, rows, cols, seed, d_lo=1e-3, d_hi=2e-2):
    el, _, _ = GEOM[ty]
    assert cols % el == 0
    return blocks(ty, rows * (cols // el), seed, d_lo, d_hi)


def bf16_normal(rows, cols, seed, std):
    """bf16 N(0, std) matrix as raw little-endian bytes (router weights): f32 normal truncated to bf16 by RNE."""
    x = (np.random.Generator(np.random.PCG64(seed)).standard_normal((rows, cols), dtype=np.float32) * np.float32(std))
    u = x.view(np.uint32)
    r = ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)
    return r.view(np.uint8).reshape(-1).copy()


def normal(shape, seed, std=1.0, mean=0.0):
    g = np.random.Generator(np.random.PCG64(seed))
    return (g.standard_normal(shape, dtype=np.float32) * np.float32(std) + np.float32(mean)).astype(np.float32)


def uniform(shape, seed, lo, hi):
    g = np.random.Generator(np.random.PCG64(seed))
    return (g.random(shape, dtype=np.float32) * np.float32(hi - lo) + np.float32(lo)).astype(np.float32)
