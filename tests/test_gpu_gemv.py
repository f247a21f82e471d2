"""GPU parity of the quantizers, the upload repack, the row dequantizers and the decode
products against the CPU oracle, through the C ABI (via the Lisp-shaped LAUNCH).  Integer
and byte results are compared bit for bit; so are the float products, because the kernels
add a row's block terms in the CPU path's order."""
import numpy as np
import pytest

import oracle_lib as orc
from illatio_amd import synth

pytestmark = pytest.mark.gpu

TYPES = [synth.Q8_0, synth.Q4_K, synth.Q6_K, synth.Q2_K, synth.IQ2_XXS]


@pytest.fixture(scope="module")
def dev():
    from illatio_amd import hip
    return hip.open_hip(0)


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def special_activations(cols, rng):
    x = synth.activations(cols, rng)
    x[0:32] = 0.0                      # a zero Q8_0 block
    if cols >= 512:
        x[256:512] = 0.0               # a zero Q8_K block
    x[40] = -7.5                       # block maximum on a negative value
    x[70] = 3.25; x[90] = -3.25        # equal magnitudes: the first wins
    if cols >= 1280:                   # a Q8_K block's largest magnitude with both signs: the first one's sign is the scale's
        x[512 + 5] = 9.0; x[512 + 200] = -9.0
        x[768 + 3] = -8.0; x[768 + 100] = 8.0; x[768 + 101] = 8.0
        x[1024 + 255] = -6.5; x[1024 + 254] = 6.5; x[1024 + 17] = 6.5
    return x


@pytest.mark.parametrize("n", [32, 2560, 4864, 32 * 1000 + 32])
def test_quant_q8_bit_exact(dev, n):
    from illatio_amd import hip
    rng = synth.make_rng(n)
    x = special_activations(n, rng) if n >= 128 else synth.activations(n, rng)
    xb = hip.hip_upload_new(dev, x)
    for f16 in (True, False):
        q, s, sm = hip.hip_alloc(dev, n), hip.hip_alloc(dev, 4 * n // 32), hip.hip_alloc(dev, 4 * n // 32)
        if f16:
            hip.launch(dev, "quant_q8", (n + 255) // 256, 256, [xb, q, s, sm, hip.I64(n // 32)])
        else:
            hip.launch(dev, "d4_quant", (n + 255) // 256, 256, [xb, q, s, n // 32])
        wq, ws = orc.quantize_q8(x, f16)
        assert np.array_equal(hip.hip_download(q, np.int8, n), wq)
        assert np.array_equal(bits(hip.hip_floats(s, n // 32)), bits(ws))
        if f16:
            assert np.array_equal(hip.hip_download(sm, np.int32, n // 32), wq.astype(np.int32).reshape(-1, 32).sum(axis=1))
        for b in (q, s, sm):
            hip.hip_free(b)
    hip.hip_free(xb)


@pytest.mark.parametrize("n", [256, 2560, 9728, 256 * 96])
def test_quant_q8k_bit_exact(dev, n):
    from illatio_amd import hip
    rng = synth.make_rng(n + 1)
    x = special_activations(n, rng)
    xb = hip.hip_upload_new(dev, x)
    q, d, bs = hip.hip_alloc(dev, n), hip.hip_alloc(dev, 4 * n // 256), hip.hip_alloc(dev, 4 * n // 16)
    hip.launch(dev, "quant_q8k", n // 256, 256, [xb, q, d, bs, hip.I64(n // 256)])
    wq, wd, wbs = orc.quantize_q8k(x)
    assert np.array_equal(hip.hip_download(q, np.int8, n), wq)
    assert np.array_equal(bits(hip.hip_floats(d, n // 256)), bits(wd))
    assert np.array_equal(hip.hip_download(bs, np.int32, n // 16), wbs)
    for b in (xb, q, d, bs):
        hip.hip_free(b)


@pytest.mark.parametrize("n", [256, 9728, 256 * 96])
def test_swiglu_quant_q8k_is_swiglu_then_quant_q8k(dev, n):
    """The gated activations of a prompt chunk quantized in the launch that makes them: the blocks of "swiglu" followed
    by "quant_q8k", which are the oracle's of its own swiglu (gates large enough for e^-x to overflow, zeros, a block
    of zeros among them)."""
    import ctypes as C
    from illatio_amd import hip
    rng = synth.make_rng(n + 7)
    g, u = special_activations(n, rng) * 3.0, special_activations(n, rng)
    g[:3] = (-200.0, 120.0, 0.0)
    if n > 512:
        u[256:512] = 0.0
    gb, ub = hip.hip_upload_new(dev, g), hip.hip_upload_new(dev, u)
    outs = []
    for fused in (True, False):
        q, d, bs = hip.hip_alloc(dev, n), hip.hip_alloc(dev, 4 * n // 256), hip.hip_alloc(dev, 4 * n // 16)
        if fused:
            hip.call("ilt_swiglu_quant_q8k", C.c_uint64(dev.stream), C.c_uint64(gb.ptr), C.c_uint64(ub.ptr), C.c_uint64(q.ptr), C.c_uint64(d.ptr),
                     C.c_uint64(bs.ptr), C.c_int64(n // 256))
            assert np.array_equal(bits(hip.hip_floats(gb, n)), bits(g))            # the gates are left as they came
        else:
            hip.launch(dev, "swiglu", (n + 255) // 256, 256, [gb, ub, hip.I64(n)])
            hip.launch(dev, "quant_q8k", n // 256, 256, [gb, q, d, bs, hip.I64(n // 256)])
        outs.append((hip.hip_download(q, np.int8, n), hip.hip_floats(d, n // 256), hip.hip_download(bs, np.int32, n // 16)))
        for b in (q, d, bs):
            hip.hip_free(b)
    wq, wd, wbs = orc.quantize_q8k(orc.swiglu(g, u))
    for got in outs:
        assert np.array_equal(got[0], wq) and np.array_equal(bits(got[1]), bits(wd)) and np.array_equal(got[2], wbs)
    hip.hip_free(gb); hip.hip_free(ub)


def upload(dev, qtype, rows, cols, w):
    """The matrix as the kernels read it: Q8_0 repacked, the rest in GGUF blocks."""
    from illatio_amd import dense, hip
    if qtype in (synth.Q8_0, synth.Q4_K, synth.Q6_K):
        return dense.upload_gmat(dev, "w", qtype, rows, cols, w)
    return dense.CMat("w", qtype, rows, cols, hip.hip_upload_new(dev, w))


@pytest.mark.parametrize("qtype", TYPES)
def test_dequant_rows_bit_exact(dev, qtype):
    from illatio_amd import hip
    import ctypes as C
    rng = synth.make_rng(40 + qtype)
    rows, cols = 40, 1024
    w = synth.weights(qtype, rows, cols, rng)
    m = upload(dev, qtype, rows, cols, w)
    idx = np.array([3, 0, 39, 17, 3], np.int32)
    ib = hip.hip_upload_new(dev, idx)
    out = hip.hip_alloc(dev, 4 * len(idx) * cols)
    hip.call("ilt_dequant_rows", C.c_uint64(dev.stream), C.c_int(qtype), C.c_uint64(m.qs.ptr),
             C.c_uint64(m.d.ptr if m.d else 0), C.c_uint64(ib.ptr), C.c_int64(len(idx)), C.c_int(cols), C.c_uint64(out.ptr))
    got = hip.hip_floats(out, len(idx) * cols).reshape(len(idx), cols)
    want = orc.dequant_rows(qtype, w, cols)[idx]
    assert np.array_equal(bits(got), bits(want))
    if qtype in (synth.Q8_0, synth.Q4_K, synth.Q6_K):
        from illatio_amd import dense
        out2 = hip.hip_alloc(dev, 4 * len(idx) * cols)
        dense.embed(dev, m, ib, out2, len(idx), cols)
        assert np.array_equal(bits(hip.hip_floats(out2, len(idx) * cols).reshape(len(idx), cols)), bits(want))
        hip.hip_free(out2)
    for b in (ib, out):
        hip.hip_free(b)
    m.free()


DENSE_SHAPES = {
    synth.Q8_0: [(4864, 896), (896, 4864), (36, 64), (1, 32)],       # the benchmark's config 1, then ragged
    synth.Q4_K: [(4096, 2560), (2560, 4096), (1024, 2560), (100, 9728), (3, 256)],
    synth.Q6_K: [(1024, 2560), (2560, 9728), (64, 5120), (37, 512)],
}


@pytest.mark.parametrize("qtype", [synth.Q8_0, synth.Q4_K, synth.Q6_K])
def test_dense_gemv_matches_cpu_path_bit_for_bit(dev, qtype):
    from illatio_amd import dense, hip
    for rows, cols in DENSE_SHAPES[qtype]:
        rng = synth.make_rng(1000 * qtype + rows + cols)
        w = synth.weights(qtype, rows, cols, rng)
        x = special_activations(cols, rng) if cols >= 512 else synth.activations(cols, rng)
        bias = synth.activations(rows, rng)
        m = upload(dev, qtype, rows, cols, w)
        act = dense.QAct(dev, 1, cols, ("q8",) if qtype == synth.Q8_0 else ("q8k",))
        xb, bb = hip.hip_upload_new(dev, x), hip.hip_upload_new(dev, bias)
        y = hip.hip_alloc(dev, 4 * rows)
        dense.quantize_act(dev, xb, act)
        dense.cmat_mul(dev, m, act, y)
        want = orc.matmul(qtype, w, rows, cols, x)
        got = hip.hip_floats(y, rows)
        assert np.array_equal(bits(got), bits(want)), (qtype, rows, cols, np.abs(got - want).max())
        # + bias, then accumulate on top: y = (W.x + b) + (W.x + b)
        dense.cmat_mul(dev, m, act, y, bias=bb)
        wb = want + bias
        assert np.array_equal(bits(hip.hip_floats(y, rows)), bits(wb))
        dense.cmat_mul(dev, m, act, y, bias=bb, acc=True)
        assert np.array_equal(bits(hip.hip_floats(y, rows)), bits(wb + wb))
        for b in (xb, bb, y):
            hip.hip_free(b)
        act.free(); m.free()


def test_d4_mvq8_grouped_rows(dev):
    """Row r against the activations of group r / group_rows (ds4f.cu:50-62)."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(77)
    rows, cols, groups = 96, 256, 3
    w = synth.weights(synth.Q8_0, rows, cols, rng)
    x = synth.activations((groups, cols), rng)
    m = upload(dev, synth.Q8_0, rows, cols, w)
    xb = hip.hip_upload_new(dev, x)
    q, s = hip.hip_alloc(dev, groups * cols), hip.hip_alloc(dev, 4 * groups * cols // 32)
    y = hip.hip_alloc(dev, 4 * rows)
    hip.launch(dev, "d4_quant", (groups * cols + 255) // 256, 256, [xb, q, s, groups * cols // 32])
    hip.launch(dev, "d4_mvq8", (rows + 3) // 4, 128, [rows, cols, rows // groups, m.qs, m.d, q, s, y])
    got = hip.hip_floats(y, rows)
    gr = rows // groups
    for g in range(groups):
        want = orc.matmul(synth.Q8_0, w[g * gr:(g + 1) * gr], gr, cols, x[g], f16_scale=False)
        assert np.array_equal(bits(got[g * gr:(g + 1) * gr]), bits(want))
    for b in (xb, q, s, y):
        hip.hip_free(b)
    m.free()


@pytest.mark.parametrize("qtype,rows,cols", [(synth.IQ2_XXS, 2048, 4096), (synth.Q2_K, 4096, 2048),
                                              (synth.IQ2_XXS, 50, 512), (synth.Q2_K, 9, 256)])
def test_indexed_expert_gemv_bit_for_bit(dev, qtype, rows, cols):
    """ptrs[z] + add addressing, per-z activations (x_stride) and outputs (y_stride)."""
    from illatio_amd import hip
    rng = synth.make_rng(qtype * 7 + rows)
    nexp, nz = 5, 3
    rb = synth.row_bytes(qtype, cols)
    pad = 512
    slot = (pad + rows * rb + 255) // 256 * 256
    w = synth.weights(qtype, nexp * rows, cols, rng).reshape(nexp, rows * rb)
    host = np.zeros((nexp, slot), np.uint8)
    host[:, pad:pad + rows * rb] = w
    pool = hip.hip_upload_new(dev, host)
    chosen = [4, 0, 2]
    ptrs = hip.hip_upload_new(dev, np.array([pool.ptr + e * slot for e in chosen], np.uint64))
    for x_stride in (0, cols):
        x = special_activations(cols * nz, rng).reshape(nz, cols) if cols >= 512 else synth.activations((nz, cols), rng)
        xb = hip.hip_upload_new(dev, x)
        kq, kd, ks = hip.hip_alloc(dev, nz * cols), hip.hip_alloc(dev, 4 * nz * cols // 256), hip.hip_alloc(dev, 4 * nz * cols // 16)
        hip.launch(dev, "quant_q8k", nz * cols // 256, 256, [xb, kq, kd, ks, hip.I64(nz * cols // 256)])
        y = hip.hip_alloc(dev, 4 * nz * rows)
        name = "d4_mvq_iq2_xxs" if qtype == synth.IQ2_XXS else "d4_mvq_q2_k"     # (activations quantized beforehand)
        hip.launch(dev, name, ((rows + 7) // 8, 1, nz), 64,
                   [cols, rows, rb, hip.I64(pad), x_stride, rows, ptrs, None, kq, y, kd, ks])
        got = hip.hip_floats(y, nz * rows).reshape(nz, rows)
        for z, e in enumerate(chosen):
            want = orc.matmul(qtype, w[e].reshape(rows, rb), rows, cols, x[z if x_stride else 0])
            assert np.array_equal(bits(got[z]), bits(want)), (qtype, z, np.abs(got[z] - want).max())
            # the x86 float order of the same integer sums (avx2.lisp:77-150), which the reference's CPUs
            # take when they compute an expert: other roundings, within 1e-5 of the largest output and of
            # each row's sum of |terms| (the yardstick of inspect/iquant-test.lisp:50-53)
            xz = x[z if x_stride else 0]
            hq, hd, hs = orc.quantize_q8k(xz)
            wrows = w[e].reshape(rows, rb)
            avx = np.array([orc.row_dot(qtype, wrows[r], cols, hq, hd, hs, order="avx2") for r in range(rows)], np.float32)
            terms = np.abs(orc.dequant_rows(qtype, wrows, cols).astype(np.float64)) @ np.abs(
                hq.astype(np.float64) * np.repeat(hd.astype(np.float64), 256))
            assert np.abs(got[z] - avx).max() <= 1e-5 * np.abs(avx).max(), (qtype, z)
            assert (np.abs(got[z].astype(np.float64) - avx) <= 1e-5 * np.maximum(terms, 1e-30)).all(), (qtype, z)
        for b in (xb, kq, kd, ks, y):
            hip.hip_free(b)
    hip.hip_free(pool); hip.hip_free(ptrs)


@pytest.mark.parametrize("qtype,rows,cols", [(synth.IQ2_XXS, 2048, 4096), (synth.Q2_K, 4096, 2048),
                                              (synth.IQ2_XXS, 50, 512), (synth.Q2_K, 9, 256)])
def test_expert_gemv_with_the_reference_arguments(dev, qtype, rows, cols):
    """d4_mv_iq2_xxs / d4_mv_q2_k launched with the reference kernels' twelve slots (ds4f.cu:769-772, 837-840):
    float rows in (quantized by the kernel as the CPU path quantizes them), ptrs[z] + add, and
    - neither counts nor bases: expert z on row z of x (DK-FFN-TAIL's launches, cuda-ds4f.lisp:937-941; x_stride 0 = all
      on one row);
    - counts and bases: expert z on rows bases[z] .. bases[z] + counts[z] - 1 (DK-FFN-SMALL's,
      cuda-ds4f-spec.lisp:83-88), an expert with no rows writing nothing, strides wider than a row;
    - srcs: an expert whose slot is empty has its matrix read through from pinned host memory into the slot first
      (ds4f.cu:742-760), and the slot holds it afterwards."""
    import ctypes
    from illatio_amd import hip
    rng = synth.make_rng(qtype * 11 + rows)
    nexp = 5
    rb = synth.row_bytes(qtype, cols)
    pad = 512
    slot = (pad + rows * rb + 255) // 256 * 256
    w = synth.weights(qtype, nexp * rows, cols, rng).reshape(nexp, rows * rb)
    host = np.zeros((nexp, slot), np.uint8)
    host[:, pad:pad + rows * rb] = w
    name = "d4_mv_iq2_xxs" if qtype == synth.IQ2_XXS else "d4_mv_q2_k"
    chosen = [4, 0, 2]
    # expert 0's slot on the device is empty; its bytes wait in pinned host memory
    dev_host = host.copy()
    dev_host[0] = 0
    pool = hip.hip_upload_new(dev, dev_host)
    pinned = hip.hip_host_alloc(dev, slot)
    ctypes.memmove(pinned, host[0].ctypes.data, slot)
    ptrs = hip.hip_upload_new(dev, np.array([pool.ptr + e * slot for e in chosen], np.uint64))
    srcs = hip.hip_upload_new(dev, np.array([0, pinned, 0], np.uint64))

    def want_row(e, xrow):
        return orc.matmul(qtype, w[e].reshape(rows, rb), rows, cols, xrow)

    # counts and bases: rows 0-1 for expert 4, rows 2-4 for expert 0 (read through), none for expert 2
    counts, bases = [2, 3, 0], [0, 2, 5]
    nrows_x = 5
    xs, ys = cols + 256, rows + 8
    x = np.zeros((nrows_x, xs), np.float32)
    x[:, :cols] = special_activations(cols * nrows_x, rng).reshape(nrows_x, cols) if cols >= 512 else synth.activations((nrows_x, cols), rng)
    xb = hip.hip_upload_new(dev, x)
    y = hip.hip_upload_new(dev, np.full(nrows_x * ys, 7.0, np.float32))
    cb, bb = hip.hip_upload_new(dev, np.array(counts, np.uint32)), hip.hip_upload_new(dev, np.array(bases, np.uint32))
    hip.launch(dev, name, ((rows + 7) // 8, 1, 3), 64, [cols, rows, rb, hip.I64(pad), xs, ys, ptrs, srcs, xb, y, cb, bb])
    got = hip.hip_floats(y, nrows_x * ys).reshape(nrows_x, ys)
    assert np.all(got[:, rows:] == 7.0)
    for z, e in enumerate(chosen):
        for r in range(bases[z], bases[z] + counts[z]):
            assert np.array_equal(bits(got[r, :rows]), bits(want_row(e, x[r, :cols]))), (qtype, z, r)
    # the slot holds the matrix now (and nothing else of the pool changed)
    back = hip.hip_download(pool, np.uint8, nexp * slot).reshape(nexp, slot)
    assert np.array_equal(back[0, pad:pad + rows * rb], w[0])
    assert np.array_equal(back[1:], host[1:])
    # with the slot filled, no srcs are needed any more
    y2 = hip.hip_upload_new(dev, np.full(nrows_x * ys, 7.0, np.float32))
    hip.launch(dev, name, ((rows + 7) // 8, 1, 3), 64, [cols, rows, rb, hip.I64(pad), xs, ys, ptrs, None, xb, y2, cb, bb])
    assert np.array_equal(bits(hip.hip_floats(y2, nrows_x * ys)), bits(got.reshape(-1)))
    # no counts: expert z on row z, or all on row 0
    for x_stride in (0, cols):
        xz = np.ascontiguousarray(x[:3, :cols])
        xzb = hip.hip_upload_new(dev, xz)
        y3 = hip.hip_alloc(dev, 4 * 3 * rows)
        hip.launch(dev, name, ((rows + 7) // 8, 1, 3), 64, [cols, rows, rb, hip.I64(pad), x_stride, rows, ptrs, None, xzb, y3, None, None])
        got3 = hip.hip_floats(y3, 3 * rows).reshape(3, rows)
        for z, e in enumerate(chosen):
            assert np.array_equal(bits(got3[z]), bits(want_row(e, xz[z if x_stride else 0]))), (qtype, z, x_stride)
        hip.hip_free(xzb); hip.hip_free(y3)
    # one of counts / bases without the other is refused
    with pytest.raises(hip.HipError):
        hip.launch(dev, name, ((rows + 7) // 8, 1, 3), 64, [cols, rows, rb, hip.I64(pad), xs, ys, ptrs, None, xb, y2, cb, None])
    hip.hip_sync(dev)
    for b in (pool, ptrs, srcs, xb, y, y2, cb, bb):
        hip.hip_free(b)
    hip.hip_host_free(pinned)


def test_d4_mvq8n_tokens_of_a_speculative_step(dev):
    """d4_mvq8n (ds4f.cu:66-107): up to nine tokens through the grouped Q8_0 product, token t's
    input x_tstride and output y_tstride apart, each token's sums decode's; no tokens write nothing."""
    from illatio_amd import hip
    rng = synth.make_rng(79)
    rows, cols, groups, ntok = 192, 512, 2, 9
    xts, yts = groups * cols + 64, rows + 5                      # strides wider than a token's data
    w = synth.weights(synth.Q8_0, rows, cols, rng)
    x = np.zeros((ntok, xts), np.float32)
    x[:, :groups * cols] = synth.activations((ntok, groups * cols), rng)
    m = upload(dev, synth.Q8_0, rows, cols, w)
    xb = hip.hip_upload_new(dev, x)
    q, s = hip.hip_alloc(dev, ntok * xts), hip.hip_alloc(dev, 4 * ntok * xts // 32)
    y = hip.hip_upload_new(dev, np.full(ntok * yts, 7.0, np.float32))
    hip.launch(dev, "d4_quant", (ntok * xts + 255) // 256, 256, [xb, q, s, ntok * xts // 32])
    hip.launch(dev, "d4_mvq8n", (rows + 3) // 4, 128, [rows, cols, rows // groups, 0, xts, yts, m.qs, m.d, q, s, y])
    assert np.all(hip.hip_floats(y, ntok * yts) == 7.0)
    for nt in (1, ntok):
        hip.launch(dev, "d4_mvq8n", (rows + 3) // 4, 128, [rows, cols, rows // groups, nt, xts, yts, m.qs, m.d, q, s, y])
        got = hip.hip_floats(y, ntok * yts).reshape(ntok, yts)
        gr = rows // groups
        for t in range(nt):
            for g in range(groups):
                want = orc.matmul(synth.Q8_0, w[g * gr:(g + 1) * gr], gr, cols, x[t, g * cols:(g + 1) * cols], f16_scale=False)
                assert np.array_equal(bits(got[t, g * gr:(g + 1) * gr]), bits(want)), (nt, t, g)
        assert np.all(got[:, rows:] == 7.0) and np.all(got[nt:] == 7.0)
    with pytest.raises(hip.HipError):
        hip.launch(dev, "d4_mvq8n", (rows + 3) // 4, 128, [rows, cols, rows // groups, 10, xts, yts, m.qs, m.d, q, s, y])
    for b in (xb, q, s, y):
        hip.hip_free(b)
    m.free()


def test_invalid_arguments_are_errors_not_faults(dev):
    from illatio_amd import hip
    b = hip.hip_alloc(dev, 4096)
    with pytest.raises(hip.HipError):
        hip.launch(dev, "mv_q8", 1, 128, [b, b, b, b, b, None, 4, 48, 0])        # cols not a multiple of 32
    with pytest.raises(hip.HipError):
        hip.launch(dev, "mv_k", 1, 128, [1, b, b, b, b, b, None, 4, 256, 0])      # Q5_K is not built
    with pytest.raises(hip.HipError):
        hip.launch(dev, "no_such_kernel", 1, 1, [])
    with pytest.raises(hip.HipError):
        hip.launch(dev, "mv_q8", 1, 128, [None, b, b, b, b, None, 4, 32, 0])      # null weights
    hip.hip_free(b)


@pytest.mark.parametrize("kind", ["k", "q8"])
def test_fused_launches_match_single_products(dev, kind):
    """Q, K, V in one launch; gate and up ending in swiglu!; and the same with the kernel
    quantizing the float activations itself -- all with the single products' bits."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(555 if kind == "k" else 556)
    cols = 2560 if kind == "k" else 896
    shapes = [(synth.Q4_K, 4096), (synth.Q4_K, 1024), (synth.Q6_K, 1024)] if kind == "k" else \
             [(synth.Q8_0, 896), (synth.Q8_0, 128), (synth.Q8_0, 132)]
    ws = [synth.weights(t, r, cols, rng) for t, r in shapes]
    ms = [upload(dev, t, r, cols, w) for (t, r), w in zip(shapes, ws)]
    x = special_activations(cols, rng)
    xb = hip.hip_upload_new(dev, x)
    act = dense.QAct(dev, 1, cols, ("q8k",) if kind == "k" else ("q8",))
    dense.quantize_act(dev, xb, act)
    biases = [None, synth.activations(shapes[1][1], rng), None]
    bbs = [None if b is None else hip.hip_upload_new(dev, b) for b in biases]
    want = [orc.matmul(t, w, r, cols, x) + (0 if b is None else b) for (t, r), w, b in zip(shapes, ws, biases)]
    for xf in (None, xb):
        ys = [hip.hip_alloc(dev, 4 * r) for _, r in shapes]
        dense.qkv_mul(dev, ms[0], ms[1], ms[2], act, ys[0], ys[1], ys[2], bbs[0], bbs[1], bbs[2], xf=xf)
        for y, wv, (_, r) in zip(ys, want, shapes):
            assert np.array_equal(bits(hip.hip_floats(y, r)), bits(wv)), ("qkv", kind, xf is not None)
        for y in ys:
            hip.hip_free(y)
    # gate/up: two matrices of equal rows (mixed K-quant formats allowed)
    gshape = [(synth.Q4_K, 1000), (synth.Q6_K, 1000)] if kind == "k" else [(synth.Q8_0, 500), (synth.Q8_0, 500)]
    gw = [synth.weights(t, r, cols, rng) for t, r in gshape]
    gm = [upload(dev, t, r, cols, w) for (t, r), w in zip(gshape, gw)]
    g = orc.matmul(gshape[0][0], gw[0], gshape[0][1], cols, x)
    u = orc.matmul(gshape[1][0], gw[1], gshape[1][1], cols, x)
    g[:3] = g[:3]  # values as they come; the extreme gates are covered below
    wglu = orc.swiglu(g, u)
    for xf in (None, xb):
        fa = hip.hip_alloc(dev, 4 * gshape[0][1])
        dense.glu_mul(dev, gm[0], gm[1], act, fa, xf=xf)
        assert np.array_equal(bits(hip.hip_floats(fa, gshape[0][1])), bits(wglu)), ("glu", kind, xf is not None)
        hip.hip_free(fa)
    for b in [xb] + [b for b in bbs if b is not None]:
        hip.hip_free(b)
    act.free()
    for m in ms + gm:
        m.free()


def test_in_kernel_quantization_single_matrix(dev):
    """xf: the float activations quantized by every workgroup as quantize-q8k! / quantize-q8!."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(909)
    for qtype, rows, cols in ((synth.Q6_K, 2560, 9728), (synth.Q4_K, 64, 256), (synth.Q8_0, 896, 4864), (synth.Q8_0, 8, 32)):
        w = synth.weights(qtype, rows, cols, rng)
        x = special_activations(cols, rng) if cols >= 512 else synth.activations(cols, rng)
        m = upload(dev, qtype, rows, cols, w)
        xb, y = hip.hip_upload_new(dev, x), hip.hip_alloc(dev, 4 * rows)
        for f16 in ((True, False) if qtype == synth.Q8_0 else (True,)):
            dense.mv_multi(dev, [(m, y, None)], xf=xb, f16_scale=f16)
            want = orc.matmul(qtype, w, rows, cols, x, f16_scale=f16)
            assert np.array_equal(bits(hip.hip_floats(y, rows)), bits(want)), (qtype, rows, cols, f16)
        hip.hip_free(xb); hip.hip_free(y); m.free()


# ---- rmsnorm! fused with the quantizers and with the products ---------------------------------

def tie_row(n):
    """A row whose mean square lies exactly between two floats (half the values a, half b with
    fl(a*a) and fl(b*b) an odd number of float steps apart): the parallel sum's check cannot
    clear it, so the kernel adds the squares again in the CPU's order."""
    f32 = np.float32
    a = f32(1.0)
    A = f32(a * a)
    b = a
    while True:
        b = np.nextafter(b, f32(2))
        B = f32(b * b)
        steps = int(B.view(np.uint32)) - int(A.view(np.uint32))
        if steps % 2 == 1:
            break
    x = np.empty(n, f32)
    x[0::2], x[1::2] = a, b
    mid = (np.float64(A) + np.float64(B)) / 2
    assert f32(mid) != f32(np.nextafter(mid, 0)) or f32(mid) != f32(np.nextafter(mid, 4))    # a rounding tie
    return x


def norm_rows(dim, n, rng):
    x = np.stack([synth.activations(dim, rng) * s for s in np.resize([1.0, 1e-3, 40.0], n)]).astype(np.float32)
    x[0, : dim // 2] *= np.float32(1e-5)          # a wide spread inside a row
    if n > 2:
        x[2] = tie_row(dim)
    if n > 3:
        x[3] = 0.0
    return x


@pytest.mark.parametrize("dim", [256, 1024, 2560, 5120, 8192])
def test_rmsnorm_quantized_bit_exact(dev, dim):
    """rmsnorm_q8 / rmsnorm_q8k: floats, quants, scales and sums are rmsnorm! then quantize-q8! /
    quantize-q8k!'s, whether the squares are added in parallel (checked) or one after another."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(dim + 5)
    n, eps = 5, 1e-6
    x = norm_rows(dim, n, rng)
    w = (synth.activations(dim, rng) * 0.2 + 1.0).astype(np.float32)
    xb, wb, hb = hip.hip_upload_new(dev, x), hip.hip_upload_new(dev, w), hip.hip_alloc(dev, 4 * n * dim)
    act = dense.QAct(dev, n, dim)
    want_h = np.stack([orc.rmsnorm(x[t], w, eps) for t in range(n)])
    q8, s8 = orc.quantize_q8(want_h)
    qk, dk, bk = orc.quantize_q8k(want_h)
    for exact_order in (False, True):
        for b in (hb, act.xq, act.xs, act.kq, act.kd, act.ksum):
            hip.hip_zero(b)
        dense.rmsnorm_q8(dev, xb, wb, act, dim, eps, n=n, h=hb, exact_order=exact_order)
        assert np.array_equal(bits(hip.hip_floats(hb, n * dim)), bits(want_h.ravel())), (dim, exact_order)
        assert np.array_equal(hip.hip_download(act.xq, np.int8, n * dim), q8)
        assert np.array_equal(bits(hip.hip_floats(act.xs, n * dim // 32)), bits(s8))
        assert np.array_equal(hip.hip_download(act.kq, np.int8, n * dim), qk)
        assert np.array_equal(bits(hip.hip_floats(act.kd, n * dim // 256)), bits(dk))
        assert np.array_equal(hip.hip_download(act.ksum, np.int32, n * dim // 16), bk)
    # launched by name as the reference launches it, with the block sums
    xsum = hip.hip_alloc(dev, 4 * n * dim // 32)
    hip.launch(dev, "rmsnorm_q8", (1, n), 256, [xb, wb, None, act.xq, act.xs, xsum, dim, float(eps)])
    assert np.array_equal(hip.hip_download(act.xq, np.int8, n * dim), q8)
    assert np.array_equal(hip.hip_download(xsum, np.int32, n * dim // 32), q8.reshape(-1, 32).astype(np.int32).sum(1))
    for b in (xb, wb, hb, xsum):
        hip.hip_free(b)
    act.free()


@pytest.mark.parametrize("kind", ["q8", "k"])
def test_norm_inside_the_product_bit_exact(dev, kind):
    """mv_multi with a norm: rmsnorm!, the quantizer and the products of Q/K/V (and gate/up with
    the gated activation) in one launch, with the bits of the three steps run one by one."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(77 if kind == "k" else 78)
    eps = 1e-6
    for cols in ((2560, 5120) if kind == "k" else (1024, 2560)):
        shape = [(synth.Q4_K, 512), (synth.Q6_K, 128), (synth.Q4_K, 136)] if kind == "k" else [(synth.Q8_0, 512), (synth.Q8_0, 128), (synth.Q8_0, 136)]
        ws = [synth.weights(t, r, cols, rng) for t, r in shape]
        ms = [upload(dev, t, r, cols, w) for (t, r), w in zip(shape, ws)]
        nw = (synth.activations(cols, rng) * 0.3 + 1.0).astype(np.float32)
        nwb = hip.hip_upload_new(dev, nw)
        for x in (synth.activations(cols, rng), tie_row(cols), norm_rows(cols, 1, rng)[0]):
            h = orc.rmsnorm(x, nw, eps)
            xb = hip.hip_upload_new(dev, x)
            ys = [hip.hip_alloc(dev, 4 * r) for _, r in shape]
            for exact_order in (False, True):
                dense.mv_multi(dev, [(m, y, None) for m, y in zip(ms, ys)], xf=xb, norm=(nwb, eps), exact_order=exact_order)
                for (t, r), w, y in zip(shape, ws, ys):
                    assert np.array_equal(bits(hip.hip_floats(y, r)), bits(orc.matmul(t, w, r, cols, h))), (kind, cols, t, exact_order)
            # gate and up (equal rows) ending in the gated activation
            fa = hip.hip_alloc(dev, 4 * shape[0][1])
            g2 = [ms[0], ms[0]] if kind == "q8" else [ms[0], upload(dev, synth.Q6_K, 512, cols, synth.weights(synth.Q6_K, 512, cols, synth.make_rng(5)))]
            u_w = ws[0] if kind == "q8" else synth.weights(synth.Q6_K, 512, cols, synth.make_rng(5))
            dense.mv_multi(dev, [(g2[0], fa, None), (g2[1], fa, None)], xf=xb, norm=(nwb, eps), glu=True)
            g = orc.matmul(shape[0][0], ws[0], 512, cols, h)
            u = orc.matmul(synth.Q8_0 if kind == "q8" else synth.Q6_K, u_w, 512, cols, h)
            assert np.array_equal(bits(hip.hip_floats(fa, 512)), bits(orc.swiglu(g, u))), (kind, cols)
            if kind == "k":
                g2[1].free()
            for b in [xb, fa] + ys:
                hip.hip_free(b)
        hip.hip_free(nwb)
        for m in ms:
            m.free()


# ---- the streamed variant of the decode product (mid-size Q4_K / Q6_K matrices) -----------------

def test_product_reading_the_next_products_rows_ahead(dev):
    """ilt_mv_multi_ahead: a layer's gate/up launch told of the down product after it (its idle waves read down's rows
    ahead into L2), Q/K/V told of wo, and a next product too small for the streamed variant: every result the plain
    call's, which is the oracle's, and the product read ahead for is right afterwards."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(777)
    d, ffn = 2560, 9728
    gw, uw, dw = synth.weights(synth.Q4_K, ffn, d, rng), synth.weights(synth.Q4_K, ffn, d, rng), synth.weights(synth.Q6_K, d, ffn, rng)
    sw = synth.weights(synth.Q6_K, 64, ffn, rng)
    gm, um, dm, sm = (dense.upload_gmat(dev, n, t, r, c, w) for n, t, r, c, w in
                      (("g", synth.Q4_K, ffn, d, gw), ("u", synth.Q4_K, ffn, d, uw), ("d", synth.Q6_K, d, ffn, dw), ("s", synth.Q6_K, 64, ffn, sw)))
    x, nw = special_activations(d, rng), (synth.activations(d, rng) * 0.2 + 1.0).astype(np.float32)
    xb, nwb = hip.hip_upload_new(dev, x), hip.hip_upload_new(dev, nw)
    fa, y, ys = hip.hip_alloc(dev, 4 * ffn), hip.hip_alloc(dev, 4 * d), hip.hip_alloc(dev, 4 * 64)
    h = orc.rmsnorm(x, nw, 1e-6)
    want_fa = orc.swiglu(orc.matmul(synth.Q4_K, gw, ffn, d, h), orc.matmul(synth.Q4_K, uw, ffn, d, h))
    for nxt in (([(dm, y, None)], False), ([(sm, ys, None)], False)):
        dense.glu_mul(dev, gm, um, None, fa, xf=xb, norm=(nwb, 1e-6), ahead=nxt)
        assert np.array_equal(bits(hip.hip_floats(fa, ffn)), bits(want_fa))
        dense.mv_multi(dev, [(dm, y, None)], xf=fa)
        assert np.array_equal(bits(hip.hip_floats(y, d)), bits(orc.matmul(synth.Q6_K, dw, d, ffn, want_fa)))
    # without a norm, onto what y holds, and told of a gate/up pair
    before = hip.hip_floats(y, d)
    dense.mv_multi(dev, [(dm, y, None)], xf=fa, acc=True, ahead=([(gm, fa, None), (um, fa, None)], True))
    assert np.array_equal(bits(hip.hip_floats(y, d)), bits(before + orc.matmul(synth.Q6_K, dw, d, ffn, want_fa)))
    for b in (xb, nwb, fa, y, ys):
        hip.hip_free(b)
    for m in (gm, um, dm, sm):
        m.free()


@pytest.mark.parametrize("stream", ["1", "0"])        # chosen by shape (these shapes qualify) / never
def test_streamed_products_bit_exact(dev, monkeypatch, stream):
    """Products of half a megabyte and more over one activation vector take the variant that streams every
    wave's rows into LDS; with it and without it the bits are the oracle's: float and
    quantized activations, one matrix, Q/K/V (Q4_K and Q6_K mixed), gate/up, bias and acc,
    ragged row counts, few and many rows per wave."""
    from illatio_amd import dense, hip
    import ctypes as C
    if stream == "0":
        monkeypatch.setenv("ILT_GEMV_STREAM", "0")
    else:
        monkeypatch.delenv("ILT_GEMV_STREAM", raising=False)
    count = hip.lib().ilt_streamed_launches
    count.restype = C.c_uint64
    before = count()
    rng = synth.make_rng(4242)
    for qtype, rows, cols in ((synth.Q4_K, 2560, 4096), (synth.Q6_K, 2560, 9728), (synth.Q6_K, 1030, 2560),
                              (synth.Q4_K, 16384, 1024), (synth.Q4_K, 3000, 12288), (synth.Q6_K, 9000, 256), (synth.Q6_K, 2000, 256),
                              (synth.Q8_0, 4864, 896), (synth.Q8_0, 896, 4864)):
        w = synth.weights(qtype, rows, cols, rng)
        x = special_activations(cols, rng)
        bias = synth.activations(rows, rng)
        m = upload(dev, qtype, rows, cols, w)
        xb, bb, y = hip.hip_upload_new(dev, x), hip.hip_upload_new(dev, bias), hip.hip_alloc(dev, 4 * rows)
        want = orc.matmul(qtype, w, rows, cols, x)
        dense.mv_multi(dev, [(m, y, None)], xf=xb)
        assert np.array_equal(bits(hip.hip_floats(y, rows)), bits(want)), (qtype, rows, cols, "float x")
        act = dense.QAct(dev, 1, cols, ("q8",) if qtype == synth.Q8_0 else ("q8k",))
        dense.quantize_act(dev, xb, act)
        dense.mv_multi(dev, [(m, y, bb)], act, acc=True)
        assert np.array_equal(bits(hip.hip_floats(y, rows)), bits(want + (want + bias))), (qtype, rows, cols, "quantized x, bias, acc")
        for b in (xb, bb, y):
            hip.hip_free(b)
        act.free(); m.free()
    # Q/K/V of a layer (two Q4_K and a Q6_K matrix in one launch) and its gate/up with the gated activation
    cols = 2560
    shape = [(synth.Q4_K, 4096), (synth.Q4_K, 1024), (synth.Q6_K, 1024)]
    ws = [synth.weights(t, r, cols, rng) for t, r in shape]
    ms = [upload(dev, t, r, cols, w) for (t, r), w in zip(shape, ws)]
    x = synth.activations(cols, rng)
    xb = hip.hip_upload_new(dev, x)
    ys = [hip.hip_alloc(dev, 4 * r) for _, r in shape]
    dense.mv_multi(dev, [(m, y, None) for m, y in zip(ms, ys)], xf=xb)
    for (t, r), w, y in zip(shape, ws, ys):
        assert np.array_equal(bits(hip.hip_floats(y, r)), bits(orc.matmul(t, w, r, cols, x))), ("qkv", t)
    gw, uw = synth.weights(synth.Q4_K, 9728, cols, rng), synth.weights(synth.Q6_K, 9728, cols, rng)
    gm, um = upload(dev, synth.Q4_K, 9728, cols, gw), upload(dev, synth.Q6_K, 9728, cols, uw)
    fa = hip.hip_alloc(dev, 4 * 9728)
    dense.glu_mul(dev, gm, um, None, fa, xf=xb)
    want = orc.swiglu(orc.matmul(synth.Q4_K, gw, 9728, cols, x), orc.matmul(synth.Q6_K, uw, 9728, cols, x))
    assert np.array_equal(bits(hip.hip_floats(fa, 9728)), bits(want)), "glu"
    # the same two launches with rmsnorm! inside: a random row, a row on a rounding tie (the sum is
    # taken again in the CPU's order), and that order forced
    nw = (synth.activations(cols, rng) * 0.3 + 1.0).astype(np.float32)
    nwb = hip.hip_upload_new(dev, nw)
    for xr, exact_order in ((x, False), (tie_row(cols), False), (x, True)):
        h = orc.rmsnorm(xr, nw, 1e-6)
        xrb = hip.hip_upload_new(dev, xr)
        dense.mv_multi(dev, [(m, y, None) for m, y in zip(ms, ys)], xf=xrb, norm=(nwb, 1e-6), exact_order=exact_order)
        for (t, r), w, y in zip(shape, ws, ys):
            assert np.array_equal(bits(hip.hip_floats(y, r)), bits(orc.matmul(t, w, r, cols, h))), ("qkv with norm", t, exact_order)
        dense.mv_multi(dev, [(gm, fa, None), (um, fa, None)], xf=xrb, norm=(nwb, 1e-6), glu=True, exact_order=exact_order)
        want = orc.swiglu(orc.matmul(synth.Q4_K, gw, 9728, cols, h), orc.matmul(synth.Q6_K, uw, 9728, cols, h))
        assert np.array_equal(bits(hip.hip_floats(fa, 9728)), bits(want)), ("glu with norm", exact_order)
        hip.hip_free(xrb)
    for b in [xb, fa, nwb] + ys:
        hip.hip_free(b)
    for m in ms + [gm, um]:
        m.free()
    # 8 shapes x 2 launches + Q/K/V + 3 x Q/K/V with the norm took the streamed variant (2000 x 256 is
    # under half a megabyte; a Q4_K gate with a Q6_K up of 9728 rows does not fit a CU's LDS)
    assert count() - before == (20 if stream == "1" else 0)
