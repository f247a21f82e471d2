"""Pins the CPU oracle (oracle/illatio_oracle.c) without running the reference: closed
forms, an independent numpy reading of the formats, brute force on integers, and the
reference's own criterion for the row dots (inspect/iquant-test.lisp:45-53: kernel vs a
double-precision dot of dequantized values, |diff| / sum|terms| < 1e-6)."""
import json
import os

import numpy as np
import pytest

import np_formats as npf
import oracle_lib as orc
from illatio_amd import synth

TYPES = [synth.Q8_0, synth.Q4_K, synth.Q6_K, synth.Q2_K, synth.IQ2_XXS]
HERE = os.path.dirname(os.path.abspath(__file__))


# ---- fp16 (half.lisp) ---------------------------------------------------------------------
def test_half_to_single_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([orc.half_to_single(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_single_to_half_rne():
    rng = synth.make_rng(11)
    halves = np.arange(0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mids = ((halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2).astype(np.float32)  # exact ties
    cand = [halves, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
            np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e10, 5.9604645e-8, 2.9802322e-8, 2.9802326e-8,
                      1e-10, 0.0, np.inf], np.float32),
            rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
            np.arange(1, 2000, dtype=np.uint32).view(np.float32)]           # single subnormals
    x = np.concatenate(cand)
    x = np.concatenate([x, -x])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([orc.single_to_half(v) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert orc.single_to_half(float("nan")) & 0x7c00 == 0x7c00 and orc.single_to_half(float("nan")) & 0x3ff


# ---- IQ2_XXS tables --------------------------------------------------------------------------
def test_iq2xxs_tables_invariants_and_headers():
    grid, signs = npf.tables()
    assert grid.size == 256 and signs.size == 128
    by = (grid[:, None] >> (np.arange(8, dtype=np.uint64) * np.uint64(8))) & np.uint64(0xFF)
    assert set(np.unique(by).tolist()) == {8, 25, 43}
    assert len(set(grid.tolist())) == 256
    for s in range(128):
        assert signs[s] == s + 128 * (bin(s).count("1") & 1)
    # both C headers carry the fixture's values
    import re
    root = os.path.dirname(HERE)
    for rel in ("oracle/iq2xxs_tables.h", "illatio_amd/csrc/ilt_iq2xxs_tables.h"):
        text = open(os.path.join(root, rel)).read()
        g = [int(h, 16) for h in re.findall(r"0x([0-9a-f]{16})ULL", text)]
        assert g == grid.tolist(), rel
        body = text[text.index("ksigns_iq2xs[128]"):]
        s = [int(v) for v in re.findall(r"\b(\d{1,3})\b", body[body.index("{"):body.index("}")])]
        assert s == signs.tolist(), rel


@pytest.mark.skipif(not os.path.isdir("/root/reference/src"), reason="reference tree not present")
def test_iq2xxs_tables_match_reference_copies():
    import importlib.util
    spec = importlib.util.spec_from_file_location("mk", os.path.join(HERE, "golden", "make_iq2xxs_tables.py"))
    mk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mk)
    grid, signs = npf.tables()
    lg, ls = mk.lisp_tables("/root/reference/src/iquant.lisp")
    assert lg == grid.tolist() and ls == signs.tolist()
    for rel in ("src/cuda/ds4f.cu", "src/metal/ds4f.metal"):
        cg, cs = mk.c_tables(os.path.join("/root/reference", rel))
        assert cg == grid.tolist() and cs[:128] == signs.tolist()


# ---- scale-min-k4 ------------------------------------------------------------------------------
def test_scale_min_k4_bitfields():
    # closed form: 8 six-bit scales then 8 six-bit mins packed in 12 bytes; the low four of
    # each live in bytes 0..7's low 6 bits, the high four split 4 bits + 2 bits.
    rng = synth.make_rng(5)
    for _ in range(300):
        sc = rng.integers(0, 64, 8)
        mn = rng.integers(0, 64, 8)
        q = np.zeros(12, np.uint8)
        for j in range(4):
            q[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
            q[j + 4] = mn[j] | ((mn[j + 4] >> 4) << 6)
            q[j + 8] = (sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4)
        for j in range(8):
            assert orc.scale_min_k4(j, q) == (sc[j], mn[j])


# ---- decoders: bit-exact against the numpy reading, and hand-built blocks ---------------------
@pytest.mark.parametrize("qtype", TYPES)
def test_dequant_matches_numpy_reading(qtype):
    rng = synth.make_rng(100 + qtype)
    cols = 512
    w = synth.weights(qtype, 24, cols, rng)
    got = orc.dequant_rows(qtype, w, cols)
    want = npf.dequant(qtype, w, cols)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def _one_hot_block(qtype):
    bb = synth.BLOCK_BYTES[qtype]
    return np.zeros((1, bb), np.uint8)


def test_dequant_hand_built_blocks():
    h1 = np.array([1.0], np.float16).view(np.uint8)       # fp16 1.0
    # Q8_0: d=1, q[5] = -3
    b = _one_hot_block(synth.Q8_0); b[0, 0:2] = h1; b[0, 2 + 5] = np.uint8(256 - 3)
    y = orc.dequant_rows(synth.Q8_0, b, 32)[0]
    assert y[5] == -3.0 and np.count_nonzero(y) == 1
    # Q4_K: d=1, scale of group 3 = 2 (byte 4+3), high nibble of qs[32*1 + 7] = 9 -> weight 64*1+32+7
    b = _one_hot_block(synth.Q4_K); b[0, 0:2] = h1; b[0, 4 + 3] = 2; b[0, 16 + 32 + 7] = 9 << 4
    y = orc.dequant_rows(synth.Q4_K, b, 256)[0]
    assert y[64 + 32 + 7] == 18.0 and np.count_nonzero(y) == 1
    # Q4_K: dmin=1, min of group 5 = 17 = 0b010001: low 4 bits in byte 4+8+1 high nibble, top 2 in byte 4+5 bits 6-7
    b = _one_hot_block(synth.Q4_K); b[0, 2:4] = h1; b[0, 4 + 9] = (17 & 0xF) << 4; b[0, 4 + 5] = (17 >> 4) << 6
    y = orc.dequant_rows(synth.Q4_K, b, 256)[0]
    assert np.all(y[160:192] == -17.0) and np.count_nonzero(y) == 32
    # Q6_K: d=1, sc[8+4+1] = -2, weight 128+64+16+3: high nibble of ql[64+16+3], bits 4-5 of qh[32+16+3]
    b = _one_hot_block(synth.Q6_K); b[0, 208:210] = h1; b[0, 192 + 13] = np.uint8(256 - 2)
    b[0, 64 + 19] = 0x5 << 4; b[0, 128 + 32 + 19] = 0x2 << 4
    y = orc.dequant_rows(synth.Q6_K, b, 256)[0]
    assert y[128 + 64 + 19] == -2.0 * ((0x5 | (0x2 << 4)) - 32)
    assert np.all(np.delete(y[128 + 64 + 16:128 + 64 + 32], 3) == -2.0 * -32)
    # Q2_K: d=1, scale byte 8+2*2+1 low nibble 3, quant (bits 4-5) of qs[32+16+9] = 2 -> weight 128+64+16+9
    b = _one_hot_block(synth.Q2_K); b[0, 80:82] = h1; b[0, 8 + 5] = 3; b[0, 16 + 32 + 16 + 9] = 2 << 4
    y = orc.dequant_rows(synth.Q2_K, b, 256)[0]
    assert y[128 + 64 + 16 + 9] == 6.0 and np.count_nonzero(y) == 1
    # IQ2_XXS: d=1, sub-block 2, LS=3, grid index 1 (=0x080808080808082b) at l=1, sign pattern 1 at l=1
    grid, signs = npf.tables()
    b = _one_hot_block(synth.IQ2_XXS); b[0, 0:2] = h1
    so = 2 + 8 * 2
    b[0, so + 1] = 1
    aux = (3 << 28) | (1 << 7)
    b[0, so + 4:so + 8] = np.array([aux], "<u4").view(np.uint8)
    y = orc.dequant_rows(synth.IQ2_XXS, b, 256)[0]
    db = np.float32(1.0) * np.float32(3.5) * np.float32(0.25)
    seg = y[64 + 8:64 + 16]
    assert seg[0] == -db * 43 and np.all(seg[1:7] == db * 8) and seg[7] == -db * 8  # ksigns[1] = 129: bits 0 and 7
    assert np.all(y[64:72] == db * 8)


# ---- quantizers ---------------------------------------------------------------------------------
def test_quantize_q8_closed_form_and_cases():
    rng = synth.make_rng(3)
    x = synth.activations(32 * 40, rng)
    x[0:32] = 0.0                                   # zero block
    x[32:64] = 0.0; x[40] = -2.5                    # single non-zero
    x[64:96] = np.arange(32, dtype=np.float32) - 16  # ties: amax 16 -> id = 127/16; 0.5*... exact halves rare
    for f16 in (True, False):
        q, s = orc.quantize_q8(x, f16)
        xb = x.reshape(-1, 32)
        amax = np.abs(xb).max(axis=1)
        d = amax / np.float32(127.0)
        with np.errstate(divide="ignore"):
            idv = np.where(d == 0, np.float32(0), np.float32(1.0) / d).astype(np.float32)
        want_q = np.rint(xb * idv[:, None]).astype(np.int8)
        assert np.array_equal(q.reshape(-1, 32), want_q)
        want_s = d.astype(np.float16).astype(np.float32) if f16 else d
        assert np.array_equal(s.view(np.uint32), want_s.view(np.uint32))
        assert np.all(q[0:32] == 0) and s[0] == 0
        assert q[40] == -127 and np.count_nonzero(q[32:64]) == 1
    # round-half-even on exact ties: d = 2/127 -> id = 63.5; x = k/127 -> x*id = k/2
    x = np.zeros(32, np.float32); x[0] = 2.0
    idv = np.float32(1.0) / (np.float32(2.0) / np.float32(127.0))
    for k in range(1, 9):
        x[k] = np.float32(k + 0.5) / idv
    q, _ = orc.quantize_q8(x, True)
    assert np.array_equal(q[1:9], np.rint((x[1:9] * idv)).astype(np.int8))


def test_quantize_q8k_closed_form_and_cases():
    rng = synth.make_rng(4)
    x = synth.activations(256 * 6, rng)
    x[0:256] = 0.0                                        # zero block: d = 0, q = 0
    x[256 + 17] = -9.0                                    # max on a negative value -> iscale positive
    x[512 + 3] = 7.0; x[512 + 200] = -7.0                 # duplicate magnitude: the first (positive) wins
    q, d, bs = orc.quantize_q8k(x)
    assert d[0] == 0 and np.all(q[0:256] == 0) and np.all(bs[0:16] == 0)
    assert q[256 + 17] == -127 and d[1] == np.float32(1.0) / (np.float32(-127.0) / np.float32(-9.0))
    assert q[512 + 3] == -127 and q[512 + 200] == 127 and d[2] < 0
    for b in range(1, 6):
        xb = x[256 * b:256 * b + 256]
        i = int(np.argmax(np.abs(xb)))                    # numpy argmax: first of equals
        isc = np.float32(-127.0) / xb[i]
        want = np.minimum(127, np.rint(isc * xb)).astype(np.int8)
        assert np.array_equal(q[256 * b:256 * b + 256], want)
        assert d[b] == np.float32(1.0) / isc
        assert np.array_equal(bs[16 * b:16 * b + 16], want.astype(np.int32).reshape(16, 16).sum(axis=1))
        assert np.max(np.abs(xb - d[b] * want.astype(np.float32))) <= abs(d[b]) * 0.5 * 1.0001 + 1e-6


# ---- integer block sums by brute force; floats against a double-precision dot ----------------------
def _quantized_act(qtype, cols, rng):
    x = (rng.random(cols, dtype=np.float32) * 2 - 1).astype(np.float32)      # U(-1,1) as iquant-test.lisp:37-38
    if qtype == synth.Q8_0:
        q, s = orc.quantize_q8(x, True)
        return x, q, s, None, np.repeat(s, 32)
    q, d, bs = orc.quantize_q8k(x)
    return x, q, d, bs, np.repeat(d, 256)


@pytest.mark.parametrize("qtype", TYPES)
def test_row_dot_integers_and_double_dot(qtype):
    rng = synth.make_rng(200 + qtype)
    cols, rows = 2048, 48
    w = synth.weights(qtype, rows, cols, rng)
    x, xq, xs, bs, xscale = _quantized_act(qtype, cols, rng)
    f = npf.decode(qtype, w, cols)
    deq = npf.dequant(qtype, w, cols).astype(np.float64)
    xi = xq.astype(np.int64)
    worst = 0.0
    for r in range(rows):
        q = f["q"][r].astype(np.int64)
        res = orc.row_dot(qtype, w[r], cols, xq, xs, bs, ints=True)
        if qtype == synth.Q8_0:
            assert np.array_equal(res[1], (q * xi).reshape(-1, 32).sum(axis=1))
        elif qtype == synth.Q4_K:
            assert np.array_equal(res[1], (q * f["isc"][r] * xi).reshape(-1, 256).sum(axis=1))
            assert np.array_equal(res[2], (f["imn"][r].astype(np.int64) * xi).reshape(-1, 256).sum(axis=1))
        elif qtype == synth.Q6_K:
            assert np.array_equal(res[1], (q * f["isc"][r] * xi).reshape(-1, 256).sum(axis=1))
            assert np.array_equal(res[2], (f["isc"][r].astype(np.int64) * xi).reshape(-1, 256).sum(axis=1))
        elif qtype == synth.Q2_K:
            assert np.array_equal(res[1], (q * f["isc"][r] * xi).reshape(-1, 256).sum(axis=1))
            assert np.array_equal(res[2], (f["imn"][r].astype(np.int64) * xi).reshape(-1, 256).sum(axis=1))
        else:
            assert np.array_equal(res[1], (q * xi).reshape(-1, 32).sum(axis=1))
        terms = deq[r] * xscale.astype(np.float64) * xi
        rel = abs(float(res[0]) - terms.sum()) / np.abs(terms).sum()
        worst = max(worst, rel)
        if qtype in (synth.Q2_K, synth.IQ2_XXS):
            v2 = orc.row_dot(qtype, w[r], cols, xq, xs, bs, order="avx2")
            assert abs(float(v2) - terms.sum()) / np.abs(terms).sum() < 1e-6
    assert worst < 1e-6, worst


def test_row_dot_sign_and_term_sensitivity():
    """A dropped min term, a wrong sign or a swapped d/dmin moves the result far beyond 1e-6:
    the double-dot check above would catch it.  Here: zero activations give zero, and scaling
    the activation scale scales the result exactly (power of two)."""
    rng = synth.make_rng(9)
    cols = 1024
    for qtype in TYPES:
        w = synth.weights(qtype, 2, cols, rng)
        x, xq, xs, bs, _ = _quantized_act(qtype, cols, rng)
        v = orc.row_dot(qtype, w[0], cols, xq, xs, bs)
        v4 = orc.row_dot(qtype, w[0], cols, xq, xs * np.float32(4.0), bs)
        assert np.float32(v4) == np.float32(v) * np.float32(4.0)
        z = orc.row_dot(qtype, w[0], cols, np.zeros_like(xq), xs, None if bs is None else np.zeros_like(bs))
        assert z == 0.0


@pytest.mark.parametrize("qtype", TYPES)
def test_matmul_is_per_token_row_dot(qtype):
    """batch.lisp:10-12: a batched product is bit-identical to one token at a time, at any thread count."""
    rng = synth.make_rng(300 + qtype)
    rows, cols, ntok = 64, 512, 5
    w = synth.weights(qtype, rows, cols, rng)
    x = synth.activations((ntok, cols), rng)
    a = orc.matmul(qtype, w, rows, cols, x, nthreads=1)
    b = orc.matmul(qtype, w, rows, cols, x, nthreads=3)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    for t in range(ntok):
        one = orc.matmul(qtype, w, rows, cols, x[t])
        assert np.array_equal(one.view(np.uint32), a[t].view(np.uint32))
    if qtype == synth.Q8_0:
        q, s = orc.quantize_q8(x[2], True)
        v = orc.row_dot(qtype, w[7], cols, q, s)
    else:
        q, d, bs = orc.quantize_q8k(x[2])
        v = orc.row_dot(qtype, w[7], cols, q, d, bs)
    assert np.float32(v) == a[2, 7]


# ---- silu / softplus: against correctly rounded values ----------------------------------------------
def test_activation_functions_correctly_rounded():
    rng = synth.make_rng(6)
    xs = np.concatenate([rng.standard_normal(4000).astype(np.float32) * 4, np.array([0, -0.0, 20, 20.5, -20, -20.5, 30, -30, 88, -88], np.float32)])
    ld = np.longdouble
    for x in xs:
        e = np.exp(ld(-abs(x)))
        sig = (ld(1) / (ld(1) + e)) if x >= 0 else e / (ld(1) + e)
        # the reference rounds exp to single first, then divides in single
        ef = np.float32(np.exp(ld(-x) if x >= 0 else ld(x)))
        want = (np.float32(1) / (np.float32(1) + ef)) if x >= 0 else ef / (np.float32(1) + ef)
        assert np.float32(orc.sigmoid(x)) == want
        assert abs(float(want) - float(sig)) <= 1.2e-7
        assert np.float32(orc.silu(x)) == np.float32(x) * want
        if x > 20:
            sp = np.float32(x)
        elif x < -20:
            sp = np.float32(np.exp(ld(x)))
        else:
            sp = np.float32(np.log(ld(np.float32(1) + np.float32(np.exp(ld(x))))))
        assert np.float32(orc.softplus(x)) == sp


# ---- swiglu! (model.lisp:364-378): x / (1 + e^-x) * b, every rounding explicit ---------------------
def test_swiglu_against_explicit_roundings_and_misreadings():
    """Each step of (* (/ x (+ 1f0 (exp (- x)))) b) rounded to single by hand from a long-double
    evaluation: exp to single (SBCL widens, calls libm, rounds back), the sum, the quotient, the
    product.  A gate below about -88.7 overflows e^-x to infinity, and the quotient is -0.0
    (model.lisp:365-368).  The d4-silu form x * sigmoid(x) (ds4f.lisp:248-251) and a product
    (x*b)/(1+e) are told apart on the same inputs."""
    f32, ld = np.float32, np.longdouble
    rng = synth.make_rng(21)
    gs = np.concatenate([rng.standard_normal(3000).astype(f32) * 5,
                         np.array([0.0, -0.0, 1.0, -1.0, 20.0, -20.0, 60.0, -60.0, 88.0, -88.0, -88.7, -88.8,
                                   -89.0, -100.0, -1000.0, 90.0, 1000.0], f32)])
    us = np.concatenate([rng.standard_normal(3000).astype(f32) * 3, rng.standard_normal(17).astype(f32)])
    got = orc.swiglu(gs, us)
    told = set()
    with np.errstate(over="ignore"):
        for x, b, y in zip(gs, us, got):
            e = f32(np.exp(ld(-x)))                              # inf past single's range
            want = f32(f32(x / f32(f32(1) + e)) * b)
            assert want.view(np.uint32) == y.view(np.uint32), (x, b)
            sig = (f32(1) / f32(f32(1) + e)) if x >= 0 else f32(np.exp(ld(x))) / f32(f32(1) + f32(np.exp(ld(x))))
            if f32(f32(x * sig) * b).view(np.uint32) != y.view(np.uint32):
                told.add("x*sigmoid")
            if f32(f32(x * b) / f32(f32(1) + e)).view(np.uint32) != y.view(np.uint32):
                told.add("(x*b)/(1+e)")
    assert told == {"x*sigmoid", "(x*b)/(1+e)"}
    # the overflow case: the quotient is minus zero, the product keeps its sign rule
    for x in (-88.8, -89.0, -100.0, -1000.0):
        for b in (2.0, -2.0):
            y = orc.swiglu([x], [b])[0]
            assert y == 0 and np.signbit(y) == (b > 0)


# ---- f32-dot16 (tensor.lisp:370-378): the router's and the attention's dot ---------------------------
def test_f32_dot16_order_against_numpy_and_misreadings():
    """Sixteen partial sums (column i into sum i mod 16, products rounded to single first), combined
    as c(j) = (s[j] + s[4+j]) + (s[8+j] + s[12+j]), (c0 + c1) + (c2 + c3): numpy's single-precision
    operations, each correctly rounded, in that order.  A plain running sum, a pairwise tree over the
    sixteen, and products kept exact (a fused multiply-add) must give other bits on some input."""
    f32 = np.float32
    rng = synth.make_rng(23)
    told = set()
    for trial in range(200):
        n = int(rng.choice([16, 32, 128, 4096]))
        a = (rng.standard_normal(n) * rng.choice([1.0, 100.0])).astype(f32)
        b = rng.standard_normal(n).astype(f32)
        s = np.zeros(16, f32)
        for j in range(0, n, 16):
            s = (s + (a[j:j + 16] * b[j:j + 16]).astype(f32)).astype(f32)
        c = [f32(f32(s[j] + s[4 + j]) + f32(s[8 + j] + s[12 + j])) for j in range(4)]
        want = f32(f32(c[0] + c[1]) + f32(c[2] + c[3]))
        got = orc.f32_dot16(a, b)
        assert got.view(np.uint32) == want.view(np.uint32), trial
        run = f32(0)
        for v in (a * b).astype(f32):
            run = f32(run + v)
        tree = s.copy()
        while tree.size > 1:
            tree = (tree[0::2] + tree[1::2]).astype(f32)
        sx = np.zeros(16, np.float64)                       # products not rounded to single before the add
        for j in range(0, n, 16):
            sx = (sx + a[j:j + 16].astype(np.float64) * b[j:j + 16].astype(np.float64)).astype(f32).astype(np.float64)
        cx = [f32(f32(f32(sx[j]) + f32(sx[4 + j])) + f32(f32(sx[8 + j]) + f32(sx[12 + j]))) for j in range(4)]
        fused = f32(f32(cx[0] + cx[1]) + f32(cx[2] + cx[3]))
        for name, v in (("running sum", run), ("pairwise tree", tree[0]), ("fused products", fused)):
            if v.view(np.uint32) != got.view(np.uint32):
                told.add(name)
    assert told == {"running sum", "pairwise tree", "fused products"}, told
    # sixteen columns: the tree alone, on values whose sums are exact
    a = np.arange(1, 17, dtype=f32); b = np.ones(16, f32)
    assert orc.f32_dot16(a, b) == 136.0
    w = rng.standard_normal((5, 64)).astype(np.float16)
    x = rng.standard_normal((3, 64)).astype(f32)
    out = orc.f16mm(w.view(np.uint16), 5, 64, x)
    for t in range(3):
        for r in range(5):
            assert out[t, r] == orc.f32_dot16(w[r].astype(f32), x[t])


# ---- routing -------------------------------------------------------------------------------------
def test_route_against_stable_sort():
    rng = synth.make_rng(7)
    for trial in range(60):
        ne, nu = (256, 6) if trial % 2 else (16, 3)
        logits = rng.standard_normal(ne).astype(np.float32)
        if trial % 3 == 0:
            logits[rng.integers(0, ne, ne // 2)] = logits[0]            # many exact ties
        bias = None if trial % 4 else (rng.standard_normal(ne).astype(np.float32) * 0.1)
        sel, w = orc.route(logits, nu, 1.5, bias)
        p = np.array([np.sqrt(np.float32(orc.softplus(v))) for v in logits], np.float32)
        s = p if bias is None else p + bias
        order = sorted(range(ne), key=lambda i: (-float(s[i]), i))[:nu]
        assert sel.tolist() == order
        tot = np.float32(0)
        for i in order:
            tot = np.float32(tot + p[i])
        want = (p[order] / tot) * np.float32(1.5)
        assert np.array_equal(w, want.astype(np.float32))
        assert abs(float(w.sum()) - 1.5) < 1e-5


def test_route_from_the_hash_table():
    """The hash layers' branch (ds4f.lisp:961-963): the token's row of tid2eid as it stands -- unsorted, the bias
    ignored -- with the weights of the other branch.  Pinned three ways: an explicit numpy evaluation with every
    rounding written out; a table row that IS the top-nu choice gives orc_route's output, which the stable sort
    pins; and the misreadings (the row sorted by score, the biased scores in the weights) give other results."""
    rng = synth.make_rng(17)
    f32 = np.float32
    for trial in range(40):
        ne, nu = (256, 6) if trial % 2 else (16, 3)
        ntok = 50
        logits = rng.standard_normal(ne).astype(f32)
        table = np.stack([rng.permutation(ne)[:nu] for _ in range(ntok)]).astype(np.int32)
        token = int(rng.integers(0, ntok))
        sel, w = orc.route_table(logits, table, token, nu, 1.5)
        assert sel.tolist() == table[token].tolist()
        p = np.array([np.sqrt(f32(orc.softplus(v))) for v in logits], f32)
        tot = f32(0)
        for i in table[token]:
            tot = f32(tot + p[i])
        tot = max(tot, f32(6.103515625e-5))
        want = ((p[table[token]] / tot) * f32(1.5)).astype(f32)
        assert np.array_equal(w.view(np.uint32), want.view(np.uint32))
        # a row equal to the top-nu choice: the other branch's output, sum order included
        tsel, tw = orc.route(logits, nu, 1.5)
        table[token] = tsel
        sel2, w2 = orc.route_table(logits, table, token, nu, 1.5)
        assert sel2.tolist() == tsel.tolist() and np.array_equal(w2.view(np.uint32), tw.view(np.uint32))
        # the row reversed: the same experts in the table's order, not by score
        table[token] = tsel[::-1]
        sel3, w3 = orc.route_table(logits, table, token, nu, 1.5)
        assert sel3.tolist() == tsel[::-1].tolist()
        assert np.allclose(w3[::-1], tw, rtol=1e-6)
    # tiny probabilities: the sum is floored at 2^-14
    logits = np.full(16, -40.0, f32)
    sel, w = orc.route_table(logits, np.array([[3, 1, 2]], np.int32), 0, 3, 1.5)
    p = np.sqrt(f32(orc.softplus(-40.0)))
    assert np.array_equal(w, np.full(3, (p / f32(6.103515625e-5)) * f32(1.5), f32))
    # an expert named twice stays twice (the table is taken as it stands)
    sel, w = orc.route_table(rng.standard_normal(16).astype(f32), np.array([[5, 5, 2]], np.int32), 0, 3, 1.5)
    assert sel.tolist() == [5, 5, 2] and w[0] == w[1]


# ---- the experts ----------------------------------------------------------------------------------
def _experts(rng, ne, d, ff):
    gate = synth.weights(synth.IQ2_XXS, ne * ff, d, rng)
    up = synth.weights(synth.IQ2_XXS, ne * ff, d, rng)
    down = synth.weights(synth.Q2_K, ne * d, ff, rng)
    return gate, up, down


def test_moe_routed_composition_and_order():
    rng = synth.make_rng(8)
    ne, d, ff, nu = 8, 512, 256, 3
    gate, up, down = _experts(rng, ne, d, ff)
    norm = synth.activations(d, rng)
    sel = np.array([5, 1, 6], np.int32)
    w = np.array([0.7, 0.5, 0.3], np.float32)
    for clamp in (0.0, 0.05):
        moe, mid = orc.moe_routed(gate, up, down, d, ff, sel, w, clamp, norm)
        xq, xd, xbs = orc.quantize_q8k(norm)
        for slot in (0, 2):
            e = sel[slot]
            for r in (0, 17, ff - 1):
                g = np.float32(orc.row_dot(synth.IQ2_XXS, gate[e * ff + r], d, xq, xd))
                u = np.float32(orc.row_dot(synth.IQ2_XXS, up[e * ff + r], d, xq, xd))
                if clamp > 1e-6:
                    g = min(g, np.float32(clamp)); u = max(np.float32(-clamp), min(u, np.float32(clamp)))
                want = (np.float32(orc.silu(g)) * u) * w[slot]
                assert mid[slot, r] == want
        for r in (0, 100, d - 1):
            acc = np.float32(0)
            for slot in range(nu):
                q, dd, bs = orc.quantize_q8k(mid[slot])
                acc = np.float32(acc + np.float32(orc.row_dot(synth.Q2_K, down[sel[slot] * d + r], ff, q, dd, bs)))
            assert moe[r] == acc
        m3, _ = orc.moe_routed(gate, up, down, d, ff, sel, w, clamp, norm, nthreads=3)
        assert np.array_equal(m3.view(np.uint32), moe.view(np.uint32))


def test_moe_chunk_equals_token_at_a_time():
    """ds4f.lisp:1128-1130: a layer-major chunk gives the decode's bits."""
    rng = synth.make_rng(10)
    ne, d, ff, nu, n = 8, 512, 256, 3, 7
    gate, up, down = _experts(rng, ne, d, ff)
    sg = synth.weights(synth.Q8_0, ff, d, rng); su = synth.weights(synth.Q8_0, ff, d, rng)
    sd = synth.weights(synth.Q8_0, d, ff, rng)
    norms = synth.activations((n, d), rng)
    logits = synth.zipf_router_logits(n, ne, rng)
    shared = np.stack([orc.moe_shared(sg, su, sd, d, ff, 0.0, norms[t]) for t in range(n)])
    out, sel, w, counts = orc.moe_chunk(gate, up, down, d, ff, ne, nu, 1.5, 0.0, logits, norms, shared, nthreads=2)
    assert counts.sum() == n * nu and np.array_equal(counts, np.bincount(sel.ravel(), minlength=ne))
    for t in range(n):
        one, s1, w1 = orc.moe_token(gate, up, down, sg, su, sd, d, ff, ne, nu, 1.5, 0.0, logits[t], norms[t])
        assert s1.tolist() == sel[t].tolist() and np.array_equal(w1, w[t])
        assert np.array_equal(one.view(np.uint32), out[t].view(np.uint32))


def test_moe_shared_composed_from_pinned_pieces():
    """d4-shared! (ds4f.lisp:1039-1048) put together by hand from functions other tests pin:
    quantize-q8! with the scale kept as a float (ds4f.lisp:1052-1053: *q8-f16-scale* NIL), the
    Q8_0 row dot, d4-silu.  The same composition with an f16-rounded scale, or with swiglu!'s
    x/(1+e^-x) in place of d4-silu, must give other bits somewhere, or the case pins nothing."""
    f32 = np.float32
    rng = synth.make_rng(22)
    d, ff = 256, 128
    sg = synth.weights(synth.Q8_0, ff, d, rng); su = synth.weights(synth.Q8_0, ff, d, rng)
    sd = synth.weights(synth.Q8_0, d, ff, rng, dscale=0.5)
    norm = synth.activations(d, rng) * f32(3)

    def compose(clamp, f16_scale, silu):
        xq, xs = orc.quantize_q8(norm, f16_scale)
        mid = np.empty(ff, f32)
        for r in range(ff):
            g = f32(orc.row_dot(synth.Q8_0, sg[r], d, xq, xs))
            u = f32(orc.row_dot(synth.Q8_0, su[r], d, xq, xs))
            if clamp > 1e-6:
                g = min(g, f32(clamp)); u = max(f32(-clamp), min(u, f32(clamp)))
            mid[r] = f32(silu(g) * u)
        mq, ms = orc.quantize_q8(mid, f16_scale)
        return np.array([orc.row_dot(synth.Q8_0, sd[r], ff, mq, ms) for r in range(d)], f32)

    d4 = lambda g: f32(orc.silu(g))
    for clamp in (0.0, 0.3):
        got = orc.moe_shared(sg, su, sd, d, ff, clamp, norm)
        want = compose(clamp, False, d4)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), clamp
        assert not np.array_equal(got.view(np.uint32), compose(clamp, True, d4).view(np.uint32))
        assert np.array_equal(got.view(np.uint32),
                              orc.moe_shared(sg, su, sd, d, ff, clamp, norm, nthreads=3).view(np.uint32))
    # the clamp changes the result on this input (it is exercised), and it is one-sided for the gate
    assert not np.array_equal(orc.moe_shared(sg, su, sd, d, ff, 0.0, norm), orc.moe_shared(sg, su, sd, d, ff, 0.3, norm))


# ---- rmsnorm! (model.lisp:205-216) -----------------------------------------------------------
# The reference holds no vector for it: these pin what its text fixes, on inputs chosen so that
# each plausible misreading (exact squares, a float sum, the weight folded into the scale,
# eps inside the mean) gives other bits.

def _rms_variants(x, w, eps):
    """The reading under test and the misreadings, in numpy with every rounding explicit."""
    f32, f64 = np.float32, np.float64
    sq = (x * x).astype(f32)                              # single-float products
    seq = f64(0)
    for s in sq:
        seq = seq + f64(s)
    n = f64(x.size)

    def out(total, order="xs"):
        scale = f32(1) / np.sqrt(f32(total / n + f64(f32(eps))))     # eps is a single float
        return ((x * scale) * w) if order == "xs" else (x * (scale * w))
    exact_sq = f64(0)
    for v in x:
        exact_sq = exact_sq + f64(v) * f64(v)
    fsum = f32(0)
    for s in sq:
        fsum = f32(fsum + s)
    return {"right": out(seq), "exact squares": out(exact_sq), "float sum": out(f64(fsum)),
            "weight folded": out(seq, "sw")}


def test_rmsnorm_closed_form_and_misreadings():
    f32 = np.float32
    # all equal powers of two: sum/n is the square itself
    x = np.full(256, 0.5, f32)
    w = np.full(256, 3.0, f32)
    want = (x * (f32(1) / np.sqrt(f32(np.float64(0.25) + np.float64(f32(1e-6)))))) * w
    assert np.array_equal(orc.rmsnorm(x, w, 1e-6).view(np.uint32), want.view(np.uint32))
    # zeros: the scale is 1/sqrt(eps), the result zeros
    assert np.array_equal(orc.rmsnorm(np.zeros(64, f32), w[:64], 1e-5), np.zeros(64, f32))
    # seeded rows until every misreading has been told apart at least once
    rng = np.random.default_rng(5)
    told = set()
    for trial in range(400):
        n = int(rng.choice([32, 64, 256, 1024]))
        x = (rng.standard_normal(n) * rng.choice([1e-3, 1.0, 30.0])).astype(f32)
        if trial % 3 == 0:
            x[: n // 2] *= f32(1e-4)                       # a wide spread of magnitudes
        w = rng.standard_normal(n).astype(f32)
        eps = float(rng.choice([1e-6, 1e-5]))
        v = _rms_variants(x, w, eps)
        got = orc.rmsnorm(x, w, eps)
        assert np.array_equal(got.view(np.uint32), v["right"].astype(f32).view(np.uint32)), trial
        for k in ("exact squares", "float sum", "weight folded"):
            if not np.array_equal(v[k].astype(f32).view(np.uint32), got.view(np.uint32)):
                told.add(k)
    assert told == {"exact squares", "float sum", "weight folded"}, told


def test_iq2xxs_even_and_odd_group_sums_are_exact_in_float():
    """The CPU path adds a block's four even (and four odd) group terms float(sumi) * (0.5 + scale)
    in single precision (iquant.lisp:161-215).  With the real codebook every such partial sum
    is a multiple of 1/2 below 2^23, so none of these additions rounds: the exact prefill kernel
    may form the integer sum of (2*scale + 1) * sumi and convert once.  The bound: four groups,
    2*15 + 1, four codebook entries a group, |quant| <= 128, the largest entry's byte sum."""
    import json, os
    tables = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "iq2xxs_tables.json")))
    grid = [int(v, 16) if isinstance(v, str) else int(v) for v in tables["iq2xxs_grid"]]
    assert len(grid) == 256 and {(g >> (8 * i)) & 0xFF for g in grid for i in range(8)} == {0x08, 0x19, 0x2B}
    largest = max(sum((g >> (8 * i)) & 0xFF for i in range(8)) for g in grid)
    assert 4 * 31 * 4 * 128 * largest < 2 ** 24          # twice the largest |partial sum|, as an integer


# ---- the dense decoder's pieces (model.lisp:205-462) ---------------------------------------------------
def test_rope_table_and_rope_head():
    """rope-table (model.lisp:218-231): theta advanced by repeated single multiplication from pos, theta-scale
    through double pow, cos and sin through double; against numpy with each rounding explicit.  A fresh power per
    pair (the misreading the reference's docstring warns of) gives other bits somewhere.  rope-head!: the pairs
    (i, i + half) when neox, (2i, 2i + 1) else, rotated by the table."""
    f32, f64 = np.float32, np.float64
    told = False
    for hd, base in ((128, 1e6), (64, 10000.0)):
        ts = f32(np.power(f64(f32(base)), f64(f32(-2.0) / f32(hd))))
        for pos in (0, 1, 7, 511, 4000):
            c, s = orc.rope_table(hd, pos, base)
            theta = f32(pos)
            for i in range(hd // 2):
                assert c[i] == f32(np.cos(f64(theta))) and s[i] == f32(np.sin(f64(theta))), (hd, pos, i)
                fresh = f32(f32(pos) * f32(np.power(f64(f32(base)), f64(f32(-2.0 * i) / f32(hd)))))
                told = told or (pos > 0 and f32(np.cos(f64(fresh))) != c[i])
                theta = f32(theta * ts)
            if pos == 0:
                assert np.all(c == 1) and np.all(s == 0)
    assert told
    x = np.arange(1, 9, dtype=f32)
    quarter = (np.zeros(4, f32), np.ones(4, f32))                   # cos 0, sin 1: (x0, x1) -> (-x1, x0)
    assert orc.rope_head(x, True, *quarter).tolist() == [-5, -6, -7, -8, 1, 2, 3, 4]
    assert orc.rope_head(x, False, *quarter).tolist() == [-2, 1, -4, 3, -6, 5, -8, 7]
    rng = synth.make_rng(31)
    v = rng.standard_normal(128).astype(f32)
    c, s = orc.rope_table(128, 77, 1e6)
    got = orc.rope_head(v, True, c, s)
    want = v.copy()
    want[:64] = (v[:64] * c).astype(f32) - (v[64:] * s).astype(f32)
    want[64:] = (v[:64] * s).astype(f32) + (v[64:] * c).astype(f32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert abs(float(np.dot(got, got)) - float(np.dot(v, v))) < 1e-3 * float(np.dot(v, v))      # a rotation


def test_attend_head_against_explicit_evaluation():
    """attend-head! (model.lisp:298-334): scores = f32-dot16 * 1/sqrt(hd); exp of a single (through double); the sum
    in double, position after position; every score times single(1/sum); out += score * V row, position after
    position.  Against numpy with each rounding explicit; a float sum or products kept exact in the output give
    other bits.  Equal keys: the mean of the values."""
    f32, f64 = np.float32, np.float64
    rng = synth.make_rng(32)
    told = set()
    for n, hd, nkv in ((1, 64, 1), (5, 64, 2), (130, 128, 2), (300, 128, 8)):
        kvd = nkv * hd
        ko = (nkv - 1) * hd
        kc, vc = rng.standard_normal((n, kvd)).astype(f32), rng.standard_normal((n, kvd)).astype(f32)
        q = (rng.standard_normal(hd) * 2).astype(f32)
        out, scores = orc.attend_head(kc, vc, q, n, hd, kvd, ko)
        scale = f32(1) / np.sqrt(f32(hd))
        sc = np.array([f32(orc.f32_dot16(kc[p, ko:ko + hd], q) * scale) for p in range(n)], f32)
        e = np.exp((sc - sc.max()).astype(f32).astype(f64)).astype(f32)
        tot, ftot = f64(0), f32(0)
        for v in e:
            tot += f64(v); ftot = f32(ftot + v)
        w = (e * f32(f64(1) / tot)).astype(f32)
        assert np.array_equal(scores.view(np.uint32), w.view(np.uint32)), n
        acc, exact = np.zeros(hd, f32), np.zeros(hd, f64)
        for p in range(n):
            acc = (acc + (w[p] * vc[p, ko:ko + hd]).astype(f32)).astype(f32)
            exact = (exact + f64(w[p]) * vc[p, ko:ko + hd].astype(f64)).astype(f32).astype(f64)
        assert np.array_equal(out.view(np.uint32), acc.view(np.uint32)), n
        if not np.array_equal((e * f32(f32(1) / ftot)).astype(f32).view(np.uint32), w.view(np.uint32)):
            told.add("float sum")
        if not np.array_equal(exact.astype(f32).view(np.uint32), out.view(np.uint32)):
            told.add("fused output")
    assert told == {"float sum", "fused output"}, told
    kc = np.tile(rng.standard_normal(64).astype(f32), (8, 1)); vc = rng.standard_normal((8, 64)).astype(f32)
    out, scores = orc.attend_head(kc, vc, rng.standard_normal(64).astype(f32), 8, 64, 64, 0)
    assert np.all(scores == f32(0.125)) and np.allclose(out, vc.mean(axis=0), atol=1e-6)


def test_forward_is_its_pieces_in_order():
    """forward-1 (model.lisp:396-462) on a tiny model, three tokens: put together by hand from the functions the
    tests above pin (rmsnorm!, the quantized products, rope, attend-head!, swiglu!), the caches included."""
    from illatio_amd import model
    f32 = np.float32
    host = model.synth_model(5, d=256, ffn=512, nh=4, nkv=2, hd=64, nl=2, vocab=300)
    c = host["config"]
    d, ffn, nh, nkv, hd = c["d"], c["ffn"], c["nh"], c["nkv"], c["hd"]
    qd, kvd = nh * hd, nkv * hd
    cpu = orc.DenseModel(host, nctx=8)
    kc, vc = np.zeros((c["nl"], 8, kvd), f32), np.zeros((c["nl"], 8, kvd), f32)
    for pos, tok in enumerate((17, 299, 0)):
        logits, xout = cpu.forward(tok, nthreads=2)
        x = orc.dequant_rows(host["embd"][0], host["embd"][1][tok:tok + 1], d)[0]
        cs, sn = orc.rope_table(hd, pos, c["rope_base"])
        for li, L in enumerate(host["layers"]):
            h = orc.rmsnorm(x, L["attn_norm"], c["eps"])
            q = orc.matmul(L["wq"][0], L["wq"][1], qd, d, h); k = orc.matmul(L["wk"][0], L["wk"][1], kvd, d, h)
            v = orc.matmul(L["wv"][0], L["wv"][1], kvd, d, h)
            for u in range(nh):
                q[u * hd:(u + 1) * hd] = orc.rope_head(orc.rmsnorm(q[u * hd:(u + 1) * hd], L["q_norm"], c["eps"]), True, cs, sn)
            for u in range(nkv):
                k[u * hd:(u + 1) * hd] = orc.rope_head(orc.rmsnorm(k[u * hd:(u + 1) * hd], L["k_norm"], c["eps"]), True, cs, sn)
            kc[li, pos], vc[li, pos] = k, v
            att = np.concatenate([orc.attend_head(kc[li], vc[li], q[u * hd:(u + 1) * hd], pos + 1, hd, kvd, (u // (nh // nkv)) * hd)[0]
                                  for u in range(nh)])
            x = (x + orc.matmul(L["wo"][0], L["wo"][1], d, qd, att)).astype(f32)
            h = orc.rmsnorm(x, L["ffn_norm"], c["eps"])
            mid = orc.swiglu(orc.matmul(L["gate"][0], L["gate"][1], ffn, d, h), orc.matmul(L["up"][0], L["up"][1], ffn, d, h))
            x = (x + orc.matmul(L["down"][0], L["down"][1], d, ffn, mid)).astype(f32)
        assert np.array_equal(xout.view(np.uint32), x.view(np.uint32)), pos
        want = orc.matmul(host["output"][0], host["output"][1], c["vocab"], d, orc.rmsnorm(x, host["output_norm"], c["eps"]))
        assert np.array_equal(logits.view(np.uint32), want.view(np.uint32)), pos
        assert np.array_equal(cpu.kc[:, :pos + 1], kc[:, :pos + 1]) and np.array_equal(cpu.vc[:, :pos + 1], vc[:, :pos + 1])
