"""Seeded synthetic GGUF-layout weights and activations for the benchmark configurations.

Nothing here reads a model file: every block is built from a counter-based
generator (numpy's Philox) in the GGUF byte order the kernels read
(block sizes as in the reference's src/gguf.lisp:33-37):

  Q8_0    34 B / 32 w   f16 d, int8 q[32]
  Q4_K   144 B / 256 w  f16 d, f16 dmin, 12 B 6-bit scales/mins, 128 B nibbles
  Q6_K   210 B / 256 w  ql[128], qh[64], int8 sc[16], f16 d
  Q2_K    84 B / 256 w  16 B scale/min nibbles, 64 B 2-bit quants, f16 d, f16 dmin
  IQ2_XXS 66 B / 256 w  f16 d, 8 x (4 grid indices, u32 signs+scale)
"""
import numpy as np

Q8_0, Q2_K, Q4_K, Q6_K, IQ2_XXS = 8, 10, 12, 14, 16
BLOCK_BYTES = {Q8_0: 34, Q2_K: 84, Q4_K: 144, Q6_K: 210, IQ2_XXS: 66}
BLOCK_WEIGHTS = {Q8_0: 32, Q2_K: 256, Q4_K: 256, Q6_K: 256, IQ2_XXS: 256}
TYPE_NAMES = {Q8_0: "q8_0", Q2_K: "q2_k", Q4_K: "q4_k", Q6_K: "q6_k", IQ2_XXS: "iq2_xxs"}


def make_rng(seed):
    return np.random.Generator(np.random.Philox(seed))


def row_bytes(qtype, cols):
    assert cols % BLOCK_WEIGHTS[qtype] == 0
    return cols // BLOCK_WEIGHTS[qtype] * BLOCK_BYTES[qtype]


def _f16_bytes(values):
    """|values| as little-endian fp16 bit patterns, shape (..., 2) uint8."""
    h = np.abs(values).astype(np.float16)
    return h.view(np.uint8).reshape(values.shape + (2,))


def weights(qtype, rows, cols, rng, dscale=None):
    """rows x cols weights of format qtype as a (rows, row_bytes) uint8 array."""
    nb = rows * (cols // BLOCK_WEIGHTS[qtype])
    bb = BLOCK_BYTES[qtype]
    blk = rng.integers(0, 256, size=(nb, bb), dtype=np.uint8)
    n = lambda: rng.standard_normal(nb).astype(np.float32)
    if qtype == Q8_0:
        blk[:, 0:2] = _f16_bytes(n() * (0.02 if dscale is None else dscale))
        q = rng.integers(-127, 128, size=(nb, 32), dtype=np.int16).astype(np.int8)
        blk[:, 2:] = q.view(np.uint8)
    elif qtype == Q4_K:
        s = 0.0005 if dscale is None else dscale
        blk[:, 0:2] = _f16_bytes(n() * s)
        blk[:, 2:4] = _f16_bytes(n() * s)
    elif qtype == Q6_K:
        blk[:, 192:208] = rng.integers(-64, 64, size=(nb, 16), dtype=np.int16).astype(np.int8).view(np.uint8)
        # (the default keeps a row's dot of a few thousand N(0,1) activations near 1; the benchmark's config 3 passes its own 0.01)
        blk[:, 208:210] = _f16_bytes(n() * (0.01 / 32.0 if dscale is None else dscale))
    elif qtype == Q2_K:
        s = 0.01 if dscale is None else dscale
        blk[:, 80:82] = _f16_bytes(n() * s)
        blk[:, 82:84] = _f16_bytes(n() * s)
    elif qtype == IQ2_XXS:
        blk[:, 0:2] = _f16_bytes(n() * (0.01 if dscale is None else dscale))
    else:
        raise ValueError(qtype)
    return blk.reshape(rows, -1)


def activations(shape, rng):
    return rng.standard_normal(shape).astype(np.float32)


def zipf_router_logits(ntok, ne, rng, alpha=1.1):
    """N(0,1) logits plus a Zipf(alpha) log-weight over a seeded expert permutation."""
    perm = rng.permutation(ne)
    logw = -alpha * np.log(np.arange(1, ne + 1, dtype=np.float64))
    bias = np.empty(ne, dtype=np.float64)
    bias[perm] = logw - logw.mean()
    return (rng.standard_normal((ntok, ne)) + bias[None, :]).astype(np.float32)
