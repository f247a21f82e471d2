"""Dense matrices on the device: the host side of the reference's src/cuda-dense.lisp for
the quantized products (UPLOAD-GMAT :75-100, CMAT-MUL :220-248, QKV-MUL :309-324), driving
the kernels through LAUNCH exactly as the Lisp host does.

Where the reference's CUDA path quantizes activations into Q8_0-style blocks for every
format, this path quantizes them as the reference's CPU path does -- Q8_0 for Q8_0
matrices, Q8_K for K-quants (matrix-act-kind, kquant.lisp:532-533) -- so results match
the CPU path bit for bit.
"""
import ctypes as C

import numpy as np

from . import hip
from .synth import BLOCK_BYTES, BLOCK_WEIGHTS, IQ2_XXS, Q2_K, Q4_K, Q6_K, Q8_0

KQUANT_CODE = {Q4_K: 0, Q6_K: 2}      # kquant-code, cuda-dense.lisp:18-20


class CMat:
    """A matrix on the device (CMAT): TYPE, ROWS, COLS, QS (and D, Q8_0's scales)."""

    def __init__(self, name, qtype, rows, cols, qs, d=None):
        self.name, self.type, self.rows, self.cols, self.qs, self.d = name, qtype, rows, cols, qs, d

    def kquant_p(self):
        return self.type in KQUANT_CODE

    def free(self):
        hip.hip_free(self.qs)
        hip.hip_free(self.d)


def upload_gmat(dev, name, qtype, rows, cols, raw_bytes):
    """RAW_BYTES (the matrix's GGUF blocks, a uint8 array) to DEV: Q8_0 split into int8s and
    scales by repack_q8; Q6_K through repack_q6k (here: 210-byte blocks padded to 212);
    Q4_K as it is."""
    if qtype not in (Q8_0, Q4_K, Q6_K):
        raise ValueError(f"the dense path multiplies Q8_0, Q4_K and Q6_K; {name} is type {qtype}")
    if cols % BLOCK_WEIGHTS[qtype]:
        raise ValueError(f"{name}: {cols} columns is not a whole number of blocks")
    raw_bytes = np.ascontiguousarray(raw_bytes, dtype=np.uint8).ravel()
    n = rows * cols
    nbytes = n // BLOCK_WEIGHTS[qtype] * BLOCK_BYTES[qtype]
    assert raw_bytes.size == nbytes
    if qtype == Q8_0:
        nb = n // 32
        raw = hip.hip_upload_new(dev, raw_bytes)
        qs, d = hip.hip_alloc(dev, n, zero=False), hip.hip_alloc(dev, 2 * nb, zero=False)
        hip.launch(dev, "repack_q8", (nb + 7) // 8, (32, 8), [raw, qs, d, hip.I64(nb)])
        hip.hip_sync(dev)
        hip.hip_free(raw)
        return CMat(name, qtype, rows, cols, qs, d)
    if qtype == Q6_K:
        nb = n // 256
        raw = hip.hip_upload_new(dev, raw_bytes)
        qs = hip.hip_alloc(dev, 224 * nb, zero=False)
        hip.launch(dev, "repack_q6k", (nb + 7) // 8, (32, 8), [raw, qs, hip.I64(nb)])
        hip.hip_sync(dev)
        hip.hip_free(raw)
        return CMat(name, qtype, rows, cols, qs)
    return CMat(name, qtype, rows, cols, hip.hip_upload_new(dev, raw_bytes))


class QAct:
    """Quantized activations on the device for N tokens of COLS: Q8_0 (xq, xs) and/or Q8_K
    (kq, kd, ksum), the formats a QACT holds (kquant.lisp:504-514)."""

    def __init__(self, dev, n, cols, kinds=("q8", "q8k")):
        self.dev, self.n, self.cols = dev, n, cols
        self.xq = self.xs = self.kq = self.kd = self.ksum = None
        if "q8" in kinds:
            self.xq, self.xs = hip.hip_alloc(dev, n * cols), hip.hip_alloc(dev, 4 * n * cols // 32)
        if "q8k" in kinds:
            self.kq, self.kd = hip.hip_alloc(dev, n * cols), hip.hip_alloc(dev, 4 * n * cols // 256)
            self.ksum = hip.hip_alloc(dev, 4 * n * cols // 16)

    def free(self):
        for b in (self.xq, self.xs, self.kq, self.kd, self.ksum):
            hip.hip_free(b)


def quantize_act(dev, x, act, n=None, f16_scale=True):
    """X (a DBuf of N x COLS floats) into ACT, in each format it holds (QUANTIZE-ACT!)."""
    n = act.n if n is None else n
    if act.xq is not None:
        nb = n * act.cols // 32
        if f16_scale:
            hip.launch(dev, "quant_q8", (nb * 32 + 255) // 256, 256, [x, act.xq, act.xs, None, hip.I64(nb)])
        else:
            hip.launch(dev, "d4_quant", (nb * 32 + 255) // 256, 256, [x, act.xq, act.xs, nb])
    if act.kq is not None:
        nb = n * act.cols // 256
        hip.launch(dev, "quant_q8k", nb, 256, [x, act.kq, act.kd, act.ksum, hip.I64(nb)])
    return act


def swiglu_quantize_act(dev, gate, up, act, n):
    """swiglu! of GATE and UP (N x COLS floats each) quantized into ACT's Q8_K blocks in one launch -- what the "swiglu"
    launch and QUANTIZE-ACT! after it leave there, without the floats written and read again; None when ACT also
    holds Q8_0 blocks (the caller then takes the two launches)."""
    if act.xq is not None or act.kq is None:
        return None
    nb = n * act.cols // 256
    hip.call("ilt_swiglu_quant_q8k", C.c_uint64(dev.stream), C.c_uint64(gate.ptr), C.c_uint64(up.ptr), C.c_uint64(act.kq.ptr),
             C.c_uint64(act.kd.ptr), C.c_uint64(act.ksum.ptr), C.c_int64(nb))
    return act


def rmsnorm_q8(dev, x, w, act, d, eps, n=1, h=None, exact_order=False):
    """RMSNORM! of N rows of X (D wide) by W, quantized into ACT in each format it holds, the
    floats into H unless None (RMSNORM-Q8, cuda-dense.lisp:260-264; Q8_K blocks when ACT holds
    them, as the CPU path makes for K-quant matrices)."""
    if act.xq is not None:
        hip.call("ilt_rmsnorm_q8", C.c_uint64(dev.stream), C.c_uint64(x.ptr), C.c_uint64(w.ptr), C.c_uint64(h.ptr if h else 0),
                 C.c_uint64(act.xq.ptr), C.c_uint64(act.xs.ptr), C.c_uint64(0), C.c_int(d), C.c_float(eps), C.c_int(n),
                 C.c_int(1 if exact_order else 0))
    if act.kq is not None:
        hip.call("ilt_rmsnorm_q8k", C.c_uint64(dev.stream), C.c_uint64(x.ptr), C.c_uint64(w.ptr), C.c_uint64(h.ptr if h else 0),
                 C.c_uint64(act.kq.ptr), C.c_uint64(act.kd.ptr), C.c_uint64(act.ksum.ptr), C.c_int(d), C.c_float(eps), C.c_int(n),
                 C.c_int(1 if exact_order else 0))
    return act


def cmat_mul(dev, w, act, y, n=1, bias=None, acc=False):
    """Y = W X for N tokens (token t's X at t*cols, its Y at t*rows), or Y += it when ACC
    (CMAT-MUL): the matrix-vector kernel for one token, the tiled product for more."""
    rows, cols = w.rows, w.cols
    a = 1 if acc else 0
    if w.kquant_p():
        code = KQUANT_CODE[w.type]
        if n == 1:
            hip.launch(dev, "mv_k", (rows + 3) // 4, 128, [code, w.qs, act.kq, act.kd, act.ksum, y, bias, rows, cols, a])
        else:
            hip.launch(dev, "mm_k", ((n + 63) // 64, (rows + 63) // 64), 256,
                       [code, w.qs, act.kq, act.kd, act.ksum, y, bias, rows, cols, n, a])
    elif n == 1:
        hip.launch(dev, "mv_q8", (rows + 3) // 4, 128, [w.qs, w.d, act.xq, act.xs, y, bias, rows, cols, a])
    else:
        hip.launch(dev, "mm_q8", ((n + 63) // 64, (rows + 63) // 64), 256,
                   [w.qs, w.d, act.xq, act.xs, y, bias, rows, cols, n, a])
    return y


BESIDE = True      # False: cmat_mul_n's launches one after another on the device's stream


def cmat_mul_n(dev, parts, act, n, acc=False):
    """PARTS, (W Y BIAS) sharing X, for N tokens (CMAT-MUL-N, cuda-dense.lisp:250-258): the K-quant matrices of one
    type, up to three at a time, in one launch of mm_k_n; whatever is left one by one."""
    todo, groups = list(parts), []
    while todo:
        w0 = todo[0][0]
        same = [pt for pt in todo if pt[0].kquant_p() and pt[0].type == w0.type and pt[0].cols == w0.cols][:3] if w0.kquant_p() and n > 1 else []
        if len(same) >= 2:
            groups.append(same)
            todo = [pt for pt in todo if not any(pt is q for q in same)]
        else:
            groups.append([todo.pop(0)])

    def run(group):
        if len(group) >= 2:
            w0 = group[0][0]
            args = [KQUANT_CODE[w0.type]]
            for k in range(3):
                w, y, bias = group[k] if k < len(group) else (None, None, None)
                args += [w.qs if w else None, y, bias, w.rows if w else 0]
            hip.launch(dev, "mm_k_n", ((n + 127) // 128, sum((w.rows + 127) // 128 for w, _, _ in group)), 512,
                       args + [act.kq, act.kd, act.ksum, w0.cols, n, 1 if acc else 0])
        else:
            w, y, bias = group[0]
            cmat_mul(dev, w, act, y, n=n, bias=bias, acc=acc)

    # A chunk's launches share X and write different Y: the ones after the first go to the device's second stream
    # (Q+K is 320 workgroups at 512 tokens and V 64: side by side they take what Q+K takes).
    if len(groups) > 1 and n > 1 and BESIDE:
        with hip.beside(dev):
            for g in groups[1:]:
                run(g)
        run(groups[0])
        hip.rejoin(dev)
    else:
        for g in groups:
            run(g)


def cvt_bf16(dev, x, n_elems, out=None):
    """N_ELEMS floats of X (a DBuf) rounded to bf16, into OUT or a new DBuf: the bf16
    product's counterpart of QUANTIZE-ACT!."""
    out = out if out is not None else hip.hip_alloc(dev, 2 * n_elems, zero=False)
    hip.launch(dev, "cvt_bf16", (n_elems // 8 + 255) // 256, 256, [x, out, hip.I64(n_elems)])
    return out


def q8k_bf16(dev, act, n, out=None, slabs=False):
    """ACT's Q8_K blocks of N tokens as bf16 -- each quant times its block's scale, the value the CPU path's row dots
    see of the activation -- as rows (for CMAT-MUL-BF16) or in slabs (for MAT-MUL-BF16): the bf16 products then share
    the CPU path's rounding of the activations to int8 blocks."""
    nbytes = slabs_bytes(n, act.cols) if slabs else 2 * n * act.cols
    out = out if out is not None else hip.hip_alloc(dev, nbytes, zero=False)
    hip.launch(dev, "q8k_bf16", 1, 256, [act.kq, act.kd, out, n, act.cols, 1 if slabs else 0])
    return out


def cmat_mul_bf16(dev, w, xb, y, n, bias=None, acc=False):
    """Y = W X for N tokens on the bf16 matrix cores, XB a DBuf of N x COLS bf16 (CVT-BF16):
    no activation quantizer runs; within 2e-2 of CMAT-MUL's result rather than equal to it."""
    if w.type not in (Q2_K, Q4_K, Q6_K, IQ2_XXS):
        raise ValueError(f"the bf16 product multiplies Q2_K, Q4_K, Q6_K and IQ2_XXS; {w.name} is type {w.type}")
    hip.launch(dev, "mm_k_bf16", ((n + 127) // 128, (w.rows + 127) // 128), 256,
               [w.type, w.qs, xb, y, bias, w.rows, w.cols, n, 1 if acc else 0])
    return y


def slabs_bytes(rows, cols):
    """Bytes of a bf16 copy in slabs of ROWS x COLS (rows padded to a multiple of 256)."""
    return 2 * cols * ((rows + 255) // 256 * 256)


def slabs_to_rows(a, rows, cols):
    """A slab copy downloaded as uint16 (32 columns of 128 rows in one piece) as ROWS x COLS."""
    g = a.reshape(-1, cols // 32, 128, 32)
    return g.transpose(0, 2, 1, 3).reshape(-1, cols)[:rows]


def dequant_bf16(dev, w, out=None):
    """The matrix W as bf16 in slabs, in OUT or a new DBuf of SLABS-BYTES, each weight the value
    CMAT-MUL-BF16 rounds inside its loop: the first pass of the two-pass product."""
    if w.type not in (Q2_K, Q4_K, Q6_K, IQ2_XXS):
        raise ValueError(f"the bf16 product multiplies Q2_K, Q4_K, Q6_K and IQ2_XXS; {w.name} is type {w.type}")
    out = out if out is not None else hip.hip_alloc(dev, slabs_bytes(w.rows, w.cols), zero=False)
    hip.launch(dev, "dequant_bf16", (w.rows + 255) // 256 * 2 * (w.cols // 128), 256, [w.type, w.qs, out, w.rows, w.cols])
    return out


def planes_bytes(rows, cols):
    """Bytes of one int8 plane of a ROWS x COLS matrix (slabs of 128 rows x 64 columns; the rows padded to a multiple of 128)."""
    return (rows + 127) // 128 * 128 * cols


def planes_to_rows(a, rows, cols):
    """A plane downloaded as bytes (64 columns of 128 rows in one piece) as ROWS x COLS."""
    return a.reshape(-1, cols // 64, 128, 64).transpose(0, 2, 1, 3).reshape(-1, cols)[:rows]


def planes_i8(dev, w, out=None):
    """The Q6_K matrix W as the exact product's two int8 planes and its d per row and
    super-block: (WH, WL, WDF), DBufs of PLANES-BYTES, PLANES-BYTES and 4*rows*cols/256 bytes
    (OUT or new ones).  The first pass of the two-pass exact product."""
    if w.type != Q6_K:
        raise ValueError(f"the planes are made of Q6_K matrices; {w.name} is type {w.type}")
    nb = planes_bytes(w.rows, w.cols)
    wh, wl, wdf = out if out is not None else (hip.hip_alloc(dev, nb), hip.hip_alloc(dev, nb), hip.hip_alloc(dev, 4 * w.rows * (w.cols // 256), zero=False))
    hip.launch(dev, "planes_i8", (w.rows * (w.cols // 256) * 16 + 255) // 256, 256, [w.type, w.qs, wh, wl, wdf, w.rows, w.cols])
    return wh, wl, wdf


def mat_mul_i8_planes(dev, planes, rows, cols, act, y, n, bias=None, acc=False):
    """Y = W X for N tokens from PLANES (PLANES-I8's result) and the Q8_K activations in ACT:
    CMAT-MUL's bits without dequantizing W again."""
    wh, wl, wdf = planes
    hip.launch(dev, "mm_i8_planes", ((n + 127) // 128, (rows + 127) // 128), 512,
               [wh, wl, wdf, act.kq, act.kd, y, bias, rows, cols, n, 1 if acc else 0])
    return y


def cvt_bf16_slabs(dev, x, n, cols, out=None):
    """N tokens of COLS floats (a DBuf) rounded to bf16 in slabs, into OUT or a new DBuf of SLABS-BYTES."""
    out = out if out is not None else hip.hip_alloc(dev, slabs_bytes(n, cols), zero=False)
    hip.launch(dev, "cvt_bf16_slabs", ((n + 255) // 256 * 256 * (cols // 8) + 255) // 256, 256, [x, out, n, cols])
    return out


def mat_mul_bf16(dev, wb, rows, cols, xs, y, n, bias=None, acc=False):
    """Y = W X for N tokens, WB the matrix (DEQUANT-BF16) and XS the activations (CVT-BF16-SLABS)
    as bf16 in slabs: the second pass."""
    hip.launch(dev, "mm_bf16", ((n + 255) // 256, (rows + 255) // 256), 256, [wb, xs, y, bias, rows, cols, n, 1 if acc else 0])
    return y


class MvDesc(C.Structure):
    _fields_ = [("gguf_type", C.c_int), ("rows", C.c_int), ("w", C.c_uint64), ("wd", C.c_uint64),
                ("y", C.c_uint64), ("bias", C.c_uint64)]


def _descs(parts):
    descs = (MvDesc * len(parts))()
    for i, (w, y, bias) in enumerate(parts):
        descs[i] = MvDesc(w.type, w.rows, w.qs.ptr, w.d.ptr if w.d else 0, y.ptr, bias.ptr if bias else 0)
    return descs


def mv_multi(dev, parts, act=None, xf=None, f16_scale=True, acc=False, glu=False, norm=None, exact_order=False, ahead=None):
    """PARTS, up to four (W Y BIAS) sharing X, in one launch (CMAT-MUL-N's idea, for one
    token): X quantized in ACT, or the floats XF, which the kernel then quantizes itself --
    after RMSNORM! by NORM = (weights DBuf, eps) when given: norm, quantizer and products in
    one launch.  AHEAD = (parts of the caller's next product, its glu flag): with float activations the launch reads
    that product's rows ahead into L2 while it runs (ilt_mv_multi_ahead)."""
    descs = _descs(parts)
    w0 = parts[0][0]
    if ahead is not None and xf is not None and not exact_order:
        nparts, nglu = ahead
        hip.call("ilt_mv_multi_ahead", C.c_uint64(dev.stream), C.c_int(len(parts)), descs, C.c_int(w0.cols), C.c_uint64(xf.ptr),
                 C.c_uint64(norm[0].ptr if norm is not None else 0), C.c_float(norm[1] if norm is not None else 0.0),
                 C.c_int(1 if f16_scale else 0), C.c_int(1 if acc else 0), C.c_int(1 if glu else 0),
                 C.c_int(len(nparts)), _descs(nparts), C.c_int(nparts[0][0].cols), C.c_int(1 if nglu else 0))
        return
    if norm is not None:
        if xf is None or acc:
            raise ValueError("a norm takes float activations and no accumulation")
        hip.call("ilt_mv_multi_norm", C.c_uint64(dev.stream), C.c_int(len(parts)), descs, C.c_int(w0.cols), C.c_uint64(xf.ptr),
                 C.c_uint64(norm[0].ptr), C.c_float(norm[1]), C.c_int(1 if exact_order else 0), C.c_int(1 if f16_scale else 0),
                 C.c_int(1 if glu else 0))
        return
    if xf is not None:
        xq = xs = bs = 0
    elif w0.kquant_p():
        xq, xs, bs = act.kq.ptr, act.kd.ptr, act.ksum.ptr
    else:
        xq, xs, bs = act.xq.ptr, act.xs.ptr, 0
    hip.call("ilt_mv_multi", C.c_uint64(dev.stream), C.c_int(len(parts)), descs, C.c_int(w0.cols), C.c_uint64(xq),
             C.c_uint64(xs), C.c_uint64(bs), C.c_uint64(xf.ptr if xf is not None else 0), C.c_int(1 if f16_scale else 0),
             C.c_int(1 if acc else 0), C.c_int(1 if glu else 0))


def qkv_mul(dev, wq, wk, wv, act, q, k, v, bq=None, bk=None, bv=None, xf=None, norm=None):
    """Q, K and V's products of one token in one launch (QKV-MUL, cuda-dense.lisp:309-324)."""
    mv_multi(dev, [(wq, q, bq), (wk, k, bk), (wv, v, bv)], act, xf, norm=norm)


def glu_mul(dev, g, u, act, fa, xf=None, norm=None, ahead=None):
    """silu(G x) * (U x) into FA for one token (GLU-MUL, cuda-dense.lisp:326-339).  AHEAD: see mv_multi."""
    if xf is not None:
        return mv_multi(dev, [(g, fa, None), (u, fa, None)], None, xf, glu=True, norm=norm, ahead=ahead)
    f, d = g.rows, g.cols
    if g.kquant_p():
        hip.launch(dev, "mv_k_glu", (f + 3) // 4, 128,
                   [KQUANT_CODE[g.type], g.qs, KQUANT_CODE[u.type], u.qs, act.kq, act.kd, act.ksum, fa, f, d])
    else:
        hip.launch(dev, "mv_q8_glu", (f + 3) // 4, 128, [g.qs, g.d, u.qs, u.d, act.xq, act.xs, fa, f, d])


def embed(dev, emb, tokens, x, n, d):
    """Rows TOKENS (a device vector of N ids) of the embedding EMB as floats in X (EMBED)."""
    if emb.kquant_p():
        hip.launch(dev, "embed_k", n, 128, [KQUANT_CODE[emb.type], emb.qs, tokens, x, d])
    else:
        hip.launch(dev, "embed_q8", n, 256, [emb.qs, emb.d, tokens, x, d])
    return x
