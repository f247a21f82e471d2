"""An independent, vectorised numpy reading of the GGUF block formats, written from the
format descriptions (ggml's dequantize_row_* loop structure), not from the oracle's C.
Used to pin the oracle's decoders and integer sums.  Test infrastructure."""
import json
import os

import numpy as np

Q8_0, Q2_K, Q4_K, Q6_K, IQ2_XXS = 8, 10, 12, 14, 16
_HERE = os.path.dirname(os.path.abspath(__file__))


def tables():
    d = json.load(open(os.path.join(_HERE, "golden", "iq2xxs_tables.json")))
    grid = np.array([int(h, 16) for h in d["iq2xxs_grid"]], dtype=np.uint64)
    signs = np.array(d["ksigns_iq2xs"], dtype=np.uint8)
    return grid, signs


def _f16(b):
    """(..., 2) uint8 -> float32 through IEEE binary16."""
    return np.ascontiguousarray(b).view(np.float16)[..., 0].astype(np.float32)


def decode(qtype, w, cols):
    """w: (rows, row_bytes) uint8.  Returns a dict of the integer fields and float scales,
    each broadcastable to (rows, cols):
       q      integer quant as the format defines it (Q6_K: 0..63, before the -32)
       scale  float multiplier of q (d, or d*sc), float32, formed as the reference forms it
       minus  float subtracted after (dmin*m), or None
       isc    integer sub-scale per weight (or None), imn integer min per weight (or None)
    """
    rows = w.shape[0]
    if qtype == Q8_0:
        blk = w.reshape(rows, cols // 32, 34)
        d = _f16(blk[..., 0:2])
        q = blk[..., 2:].view(np.int8).astype(np.int32)
        return dict(q=q.reshape(rows, cols), d=np.repeat(d, 32, axis=1), isc=None, imn=None, dmin=None)
    nb = cols // 256
    if qtype == Q4_K:
        blk = w.reshape(rows, nb, 144)
        d, dmin = _f16(blk[..., 0:2]), _f16(blk[..., 2:4])
        s = blk[..., 4:16].astype(np.int32)
        sc = np.empty((rows, nb, 8), np.int32)
        mn = np.empty((rows, nb, 8), np.int32)
        for j in range(8):
            if j < 4:
                sc[..., j] = s[..., j] & 63
                mn[..., j] = s[..., j + 4] & 63
            else:
                sc[..., j] = (s[..., j + 4] & 0xF) | ((s[..., j - 4] >> 6) << 4)
                mn[..., j] = (s[..., j + 4] >> 4) | ((s[..., j] >> 6) << 4)
        qs = blk[..., 16:].reshape(rows, nb, 4, 32).astype(np.int32)
        q = np.stack([qs & 0xF, qs >> 4], axis=3)            # (rows, nb, 4, 2, 32): chunk k, lo/hi, l
        q = q.reshape(rows, nb, 256)
        rep = lambda a: np.repeat(a, 32, axis=2)
        return dict(q=q.reshape(rows, cols), d=np.repeat(d, 256, axis=1), dmin=np.repeat(dmin, 256, axis=1),
                    isc=rep(sc).reshape(rows, cols), imn=rep(mn).reshape(rows, cols))
    if qtype == Q6_K:
        blk = w.reshape(rows, nb, 210)
        ql = blk[..., 0:128].astype(np.int32).reshape(rows, nb, 2, 64)
        qh = blk[..., 128:192].astype(np.int32).reshape(rows, nb, 2, 32)
        sc = blk[..., 192:208].view(np.int8).astype(np.int32).reshape(rows, nb, 2, 8)
        d = _f16(blk[..., 208:210])
        q = np.empty((rows, nb, 2, 128), np.int32)
        isc = np.empty((rows, nb, 2, 128), np.int32)
        l = np.arange(32)
        for n in range(2):
            a, b, h = ql[:, :, n, 0:32], ql[:, :, n, 32:64], qh[:, :, n, :]
            q[:, :, n, 0:32] = (a & 0xF) | (((h >> 0) & 3) << 4)
            q[:, :, n, 32:64] = (b & 0xF) | (((h >> 2) & 3) << 4)
            q[:, :, n, 64:96] = (a >> 4) | (((h >> 4) & 3) << 4)
            q[:, :, n, 96:128] = (b >> 4) | (((h >> 6) & 3) << 4)
            for part in range(4):
                isc[:, :, n, 32 * part:32 * part + 32] = sc[:, :, n, 2 * part + l // 16]
        return dict(q=q.reshape(rows, cols), d=np.repeat(d, 256, axis=1), isc=isc.reshape(rows, cols), imn=None, dmin=None)
    if qtype == Q2_K:
        blk = w.reshape(rows, nb, 84)
        sb = blk[..., 0:16].astype(np.int32).reshape(rows, nb, 2, 8)
        qs = blk[..., 16:80].astype(np.int32).reshape(rows, nb, 2, 32)
        d, dmin = _f16(blk[..., 80:82]), _f16(blk[..., 82:84])
        q = np.empty((rows, nb, 2, 4, 32), np.int32)
        isc = np.empty((rows, nb, 2, 4, 32), np.int32)
        imn = np.empty((rows, nb, 2, 4, 32), np.int32)
        for k in range(4):
            q[:, :, :, k, :] = (qs >> (2 * k)) & 3
            for half in range(2):
                s = sb[:, :, :, 2 * k + half]
                isc[:, :, :, k, 16 * half:16 * half + 16] = (s & 15)[..., None]
                imn[:, :, :, k, 16 * half:16 * half + 16] = (s >> 4)[..., None]
        return dict(q=q.reshape(rows, cols), d=np.repeat(d, 256, axis=1), dmin=np.repeat(dmin, 256, axis=1),
                    isc=isc.reshape(rows, cols), imn=imn.reshape(rows, cols))
    if qtype == IQ2_XXS:
        grid, ksigns = tables()
        blk = w.reshape(rows, nb, 66)
        d = _f16(blk[..., 0:2])
        sub = blk[..., 2:].reshape(rows, nb, 8, 8)
        gi = sub[..., 0:4]
        aux = np.ascontiguousarray(sub[..., 4:8]).view("<u4")[..., 0]
        ls = (aux >> 28).astype(np.int32)
        mags = ((grid[gi][..., None] >> (np.arange(8, dtype=np.uint64) * np.uint64(8))) & np.uint64(0xFF)).astype(np.int32)
        sidx = (aux[..., None] >> (7 * np.arange(4, dtype=np.uint32))) & 127
        sbits = (ksigns[sidx][..., None] >> np.arange(8, dtype=np.uint8)) & 1
        q = mags * np.where(sbits == 1, -1, 1)
        return dict(q=q.reshape(rows, cols), d=np.repeat(d, 256, axis=1), ls=np.repeat(ls.reshape(rows, nb * 8), 32, axis=1),
                    isc=None, imn=None, dmin=None)
    raise ValueError(qtype)


def dequant(qtype, w, cols):
    """float32 weights, each expression in the order ggml's dequantize_row_* uses."""
    f = decode(qtype, w, cols)
    q = f["q"].astype(np.float32)
    if qtype == Q8_0:
        return f["d"] * q
    if qtype == Q4_K or qtype == Q2_K:
        return (f["d"] * f["isc"].astype(np.float32)) * q - f["dmin"] * f["imn"].astype(np.float32)
    if qtype == Q6_K:
        return (f["d"] * f["isc"].astype(np.float32)) * (f["q"] - 32).astype(np.float32)
    if qtype == IQ2_XXS:
        db = (f["d"] * (np.float32(0.5) + f["ls"].astype(np.float32))) * np.float32(0.25)
        mag = np.abs(f["q"]).astype(np.float32)
        sgn = np.where(f["q"] < 0, np.float32(-1), np.float32(1))
        return (db * mag) * sgn
    raise ValueError(qtype)
