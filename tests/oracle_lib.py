"""ctypes binding of the CPU oracle (oracle/liboracle.so) for the tests, smoke() and the
bench's cpu_baseline leg.  Test infrastructure: the shipped library never loads this."""
import ctypes as C
import os
import subprocess

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SO = os.path.join(_ROOT, "oracle", "liboracle.so")

Q8_0, Q2_K, Q4_K, Q6_K, IQ2_XXS = 8, 10, 12, 14, 16


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", os.path.join(_ROOT, "oracle"), "-B" if force else "-s"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        L = _lib
        L.orc_half_to_single.restype = C.c_float
        L.orc_half_to_single.argtypes = [C.c_uint16]
        L.orc_single_to_half.restype = C.c_uint16
        L.orc_single_to_half.argtypes = [C.c_float]
        for name in ("orc_q8_0_row_dot", "orc_q4k_row_dot", "orc_q6k_row_dot", "orc_iq2xxs_row_dot",
                     "orc_iq2xxs_row_dot_avx2", "orc_q2k_row_dot", "orc_q2k_row_dot_avx2",
                     "orc_sigmoid", "orc_silu", "orc_softplus", "orc_swiglu"):
            getattr(L, name).restype = C.c_float
        L.orc_swiglu.argtypes = [C.c_float, C.c_float]
        for name in ("orc_sigmoid", "orc_silu", "orc_softplus"):
            getattr(L, name).argtypes = [C.c_float]
        for name in ("orc_block_bytes", "orc_block_weights"):
            getattr(L, name).restype = C.c_int64
            getattr(L, name).argtypes = [C.c_int]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def half_to_single(h):
    return lib().orc_half_to_single(int(h))


def single_to_half(x):
    return lib().orc_single_to_half(float(np.float32(x)))


def quantize_q8(x, f16_scale=True):
    x = _c(x, np.float32).ravel()
    n = x.size
    q = np.empty(n, np.int8)
    s = np.empty(n // 32, np.float32)
    lib().orc_quantize_q8(_p(x), C.c_int64(n), C.c_int(1 if f16_scale else 0), _p(q), _p(s))
    return q, s


def quantize_q8k(x):
    x = _c(x, np.float32).ravel()
    n = x.size
    q = np.empty(n, np.int8)
    d = np.empty(n // 256, np.float32)
    bs = np.empty(n // 16, np.int32)
    lib().orc_quantize_q8k(_p(x), C.c_int64(n), _p(q), _p(d), _p(bs))
    return q, d, bs


def row_dot(qtype, wrow, cols, xq, xs, bsums=None, order="neon", ints=False):
    """One row (GGUF bytes) against quantized activations; returns the float, and with
    ints=True also the exact integer block sums the reference forms on the way."""
    L = lib()
    wrow = _c(wrow, np.uint8)
    xq = _c(xq, np.int8)
    xs = _c(xs, np.float32)
    nb = cols // 256
    if qtype == Q8_0:
        acc = np.zeros(cols // 32, np.int32)
        v = L.orc_q8_0_row_dot(_p(wrow), C.c_int64(cols), _p(xq), _p(xs), _p(acc))
        return (v, acc) if ints else v
    bsums = _c(bsums, np.int32) if bsums is not None else None
    if qtype == Q4_K:
        a, b = np.zeros(nb, np.int32), np.zeros(nb, np.int32)
        v = L.orc_q4k_row_dot(_p(wrow), C.c_int64(nb), _p(xq), _p(xs), _p(bsums), _p(a), _p(b))
        return (v, a, b) if ints else v
    if qtype == Q6_K:
        a, b = np.zeros(nb, np.int32), np.zeros(nb, np.int32)
        v = L.orc_q6k_row_dot(_p(wrow), C.c_int64(nb), _p(xq), _p(xs), _p(bsums), _p(a), _p(b))
        return (v, a, b) if ints else v
    if qtype == Q2_K:
        if order == "avx2":
            return L.orc_q2k_row_dot_avx2(_p(wrow), C.c_int64(nb), _p(xq), _p(xs), _p(bsums))
        a, b = np.zeros(nb, np.int32), np.zeros(nb, np.int32)
        v = L.orc_q2k_row_dot(_p(wrow), C.c_int64(nb), _p(xq), _p(xs), _p(bsums), _p(a), _p(b))
        return (v, a, b) if ints else v
    if qtype == IQ2_XXS:
        if order == "avx2":
            return L.orc_iq2xxs_row_dot_avx2(_p(wrow), C.c_int64(nb), _p(xq), _p(xs))
        a = np.zeros(nb * 8, np.int32)
        v = L.orc_iq2xxs_row_dot(_p(wrow), C.c_int64(nb), _p(xq), _p(xs), _p(a))
        return (v, a) if ints else v
    raise ValueError(qtype)


def scale_min_k4(j, q12):
    q12 = _c(q12, np.uint8)
    sc, m = C.c_int(), C.c_int()
    lib().orc_scale_min_k4(C.c_int(j), _p(q12), C.byref(sc), C.byref(m))
    return sc.value, m.value


def dequant_rows(qtype, w, cols):
    w = _c(w, np.uint8)
    rows = w.shape[0]
    out = np.empty((rows, cols), np.float32)
    for r in range(rows):
        lib().orc_dequant_row(C.c_int(qtype), _p(w[r]), C.c_int64(cols), _p(out[r]))
    return out


def matmul(qtype, w, rows, cols, x, f16_scale=True, nthreads=1):
    """out[t, r] for x of shape (ntok, cols) (or (cols,) for one token)."""
    w = _c(w, np.uint8)
    x = _c(x, np.float32)
    ntok = 1 if x.ndim == 1 else x.shape[0]
    out = np.empty((ntok, rows), np.float32)
    lib().orc_matmul(C.c_int(qtype), _p(w), C.c_int64(rows), C.c_int64(cols), _p(x), C.c_int64(ntok),
                     C.c_int(1 if f16_scale else 0), _p(out), C.c_int(nthreads))
    return out[0] if x.ndim == 1 else out


def matmul_q(qtype, w, rows, cols, xq, xs, bsums, ntok, nthreads=1):
    w = _c(w, np.uint8)
    out = np.empty((ntok, rows), np.float32)
    lib().orc_matmul_q(C.c_int(qtype), _p(w), C.c_int64(rows), C.c_int64(cols), _p(_c(xq, np.int8)),
                       _p(_c(xs, np.float32)), _p(None if bsums is None else _c(bsums, np.int32)),
                       C.c_int64(ntok), _p(out), C.c_int(nthreads))
    return out


def f32_dot16(a, b):
    """F32-DOT16 (tensor.lisp:370-378) of two float vectors."""
    a, b = _c(a, np.float32).ravel(), _c(b, np.float32).ravel()
    f = lib().orc_f32_dot16
    f.restype = C.c_float
    return np.float32(f(_p(a), _p(b), C.c_int64(a.size)))


def f16mm(w_bits, rows, cols, x):
    """out[t, r] = F32-DOT16(W[r], x[t]) for W given as f16 bit patterns (f32mm!, ds4f.lisp:278-293)."""
    w_bits, x = _c(w_bits, np.uint16), _c(x, np.float32)
    ntok = 1 if x.ndim == 1 else x.shape[0]
    out = np.empty((ntok, rows), np.float32)
    lib().orc_f16mm(_p(w_bits), C.c_int64(rows), C.c_int64(cols), _p(x), C.c_int64(ntok), _p(out))
    return out[0] if x.ndim == 1 else out


def silu(x):
    return lib().orc_silu(float(np.float32(x)))


def sigmoid(x):
    return lib().orc_sigmoid(float(np.float32(x)))


def swiglu(g, u):
    """silu(g) * u as the dense models compute it (swiglu!, model.lisp:364-378), elementwise."""
    g = np.ascontiguousarray(g, np.float32).ravel()
    u = np.ascontiguousarray(u, np.float32).ravel()
    f = lib().orc_swiglu
    return np.array([f(float(a), float(b)) for a, b in zip(g, u)], np.float32)


def rmsnorm(x, w, eps):
    x, w = _c(x, np.float32), _c(w, np.float32)
    out = np.empty_like(x)
    lib().orc_rmsnorm(_p(x), _p(w), _p(out), C.c_float(eps), C.c_int64(x.size))
    return out


def softplus(x):
    return lib().orc_softplus(float(np.float32(x)))


def route(logits, nu, scale, bias=None):
    logits = _c(logits, np.float32)
    ne = logits.size
    sel = np.empty(nu, np.int32)
    w = np.empty(nu, np.float32)
    b = None if bias is None else _c(bias, np.float32)
    lib().orc_route(_p(logits), _p(b), C.c_int(ne), C.c_int(nu), C.c_float(scale), _p(sel), _p(w))
    return sel, w


def route_table(logits, tid2eid, token, nu, scale):
    """d4-route on a hash layer: TOKEN's row of the TID2EID table (ds4f.lisp:961-963)."""
    logits = _c(logits, np.float32)
    table = _c(tid2eid, np.int32)
    sel = np.empty(nu, np.int32)
    w = np.empty(nu, np.float32)
    lib().orc_route_table(_p(logits), _p(table), C.c_int(int(token)), C.c_int(logits.size), C.c_int(nu), C.c_float(scale),
                          _p(sel), _p(w))
    return sel, w


def moe_routed(gate, up, down, d, ff, sel, w, clamp, norm, avx2=False, nthreads=1):
    nu = len(sel)
    moe = np.empty(d, np.float32)
    mid = np.empty(nu * ff, np.float32)
    lib().orc_moe_routed(_p(_c(gate, np.uint8)), _p(_c(up, np.uint8)), _p(_c(down, np.uint8)), C.c_int(d), C.c_int(ff),
                         C.c_int(nu), _p(_c(sel, np.int32)), _p(_c(w, np.float32)), C.c_float(clamp),
                         _p(_c(norm, np.float32)), _p(moe), _p(mid), C.c_int(1 if avx2 else 0), C.c_int(nthreads))
    return moe, mid.reshape(nu, ff)


def moe_shared(sgate, sup, sdown, d, ff, clamp, norm, nthreads=1):
    out = np.empty(d, np.float32)
    lib().orc_moe_shared(_p(_c(sgate, np.uint8)), _p(_c(sup, np.uint8)), _p(_c(sdown, np.uint8)), C.c_int(d), C.c_int(ff),
                         C.c_float(clamp), _p(_c(norm, np.float32)), _p(out), C.c_int(nthreads))
    return out


def moe_token(gate, up, down, sgate, sup, sdown, d, ff, ne, nu, scale, clamp, logits, norm, bias=None,
              avx2=False, nthreads=1):
    out = np.empty(d, np.float32)
    sel = np.empty(nu, np.int32)
    w = np.empty(nu, np.float32)
    b = None if bias is None else _c(bias, np.float32)
    lib().orc_moe_token(_p(_c(gate, np.uint8)), _p(_c(up, np.uint8)), _p(_c(down, np.uint8)),
                        _p(_c(sgate, np.uint8)), _p(_c(sup, np.uint8)), _p(_c(sdown, np.uint8)),
                        C.c_int(d), C.c_int(ff), C.c_int(ne), C.c_int(nu), C.c_float(scale), C.c_float(clamp),
                        _p(_c(logits, np.float32)), _p(b), _p(_c(norm, np.float32)), _p(sel), _p(w), _p(out),
                        C.c_int(1 if avx2 else 0), C.c_int(nthreads))
    return out, sel, w


def moe_chunk(gate, up, down, d, ff, ne, nu, scale, clamp, logits, norms, shared=None, bias=None, nthreads=1):
    logits = _c(logits, np.float32)
    norms = _c(norms, np.float32)
    n = logits.shape[0]
    out = np.empty((n, d), np.float32)
    sel = np.empty((n, nu), np.int32)
    w = np.empty((n, nu), np.float32)
    counts = np.empty(ne, np.int32)
    b = None if bias is None else _c(bias, np.float32)
    sh = None if shared is None else _c(shared, np.float32)
    lib().orc_moe_chunk(_p(_c(gate, np.uint8)), _p(_c(up, np.uint8)), _p(_c(down, np.uint8)), C.c_int(d), C.c_int(ff),
                        C.c_int(ne), C.c_int(nu), C.c_float(scale), C.c_float(clamp), C.c_int(n), _p(logits), _p(b),
                        _p(norms), _p(sh), _p(out), _p(sel), _p(w), _p(counts), C.c_int(nthreads))
    return out, sel, w, counts


# ---- the dense decoder (model.lisp:205-462) ---------------------------------------------------------
def rope_table(head_dim, pos, base):
    c, s = np.empty(head_dim // 2, np.float32), np.empty(head_dim // 2, np.float32)
    lib().orc_rope_table(C.c_int(head_dim), C.c_int(pos), C.c_float(base), _p(c), _p(s))
    return c, s


def rope_head(x, neox, cosv, sinv):
    x = np.array(x, np.float32)
    lib().orc_rope_head(_p(x), C.c_int(x.size), C.c_int(1 if neox else 0), _p(_c(cosv, np.float32)), _p(_c(sinv, np.float32)))
    return x


def attend_head(kc, vc, q, n, hd, kvd, ko):
    out, scores = np.empty(hd, np.float32), np.empty(n, np.float32)
    lib().orc_attend_head(_p(_c(kc, np.float32)), _p(_c(vc, np.float32)), _p(_c(q, np.float32)), _p(out), C.c_int(n), C.c_int(hd),
                          C.c_int(kvd), C.c_int(ko), _p(scores))
    return out, scores


class _Layer(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown")] + \
               [(n, C.c_int) for n in ("tq", "tk", "tv", "to", "tg", "tu", "td")] + \
               [(n, C.c_void_p) for n in ("attn_norm", "ffn_norm", "q_norm", "k_norm", "bq", "bk", "bv")]


class _Model(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("d", "ffn", "nh", "nkv", "hd", "nl", "vocab", "neox")] + [("eps", C.c_float), ("rope_base", C.c_float),
               ("embd", C.c_void_p), ("output", C.c_void_p), ("embd_type", C.c_int), ("output_type", C.c_int), ("output_norm", C.c_void_p),
               ("layers", C.POINTER(_Layer))]


class DenseModel:
    """The CPU side of a dense decoder: HOST = a dict as illatio_amd.model.synth_model makes it (numpy arrays)."""

    def __init__(self, host, nctx):
        self.h, self.nctx = host, nctx
        c = host["config"]
        self.keep = []

        def ptr(a):
            if a is None:
                return None
            self.keep.append(a)
            return a.ctypes.data
        self.layers = (_Layer * c["nl"])()
        for i, L in enumerate(host["layers"]):
            self.layers[i] = _Layer(*[ptr(L[n][1]) for n in ("wq", "wk", "wv", "wo", "gate", "up", "down")],
                                    *[L[n][0] for n in ("wq", "wk", "wv", "wo", "gate", "up", "down")],
                                    ptr(L["attn_norm"]), ptr(L["ffn_norm"]), ptr(L.get("q_norm")), ptr(L.get("k_norm")),
                                    ptr(L.get("bq")), ptr(L.get("bk")), ptr(L.get("bv")))
        self.m = _Model(c["d"], c["ffn"], c["nh"], c["nkv"], c["hd"], c["nl"], c["vocab"], 1 if c["neox"] else 0, c["eps"], c["rope_base"],
                        ptr(host["embd"][1]), ptr(host["output"][1]), host["embd"][0], host["output"][0], ptr(host["output_norm"]), self.layers)
        kvd = c["nkv"] * c["hd"]
        self.kc = np.zeros((c["nl"], nctx, kvd), np.float32)
        self.vc = np.zeros((c["nl"], nctx, kvd), np.float32)
        self.pos = 0

    def forward(self, token, logits=True, nthreads=8):
        c = self.h["config"]
        lg = np.empty(c["vocab"], np.float32) if logits else None
        x = np.empty(c["d"], np.float32)
        lib().orc_forward(C.byref(self.m), C.c_int(int(token)), C.c_int(self.pos), _p(self.kc), _p(self.vc), C.c_int(self.nctx), _p(lg), _p(x),
                          C.c_int(nthreads))
        self.pos += 1
        return lg, x
