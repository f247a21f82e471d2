"""GPU parity of the prefill products (int8 matrix cores) with the CPU oracle, through the
C ABI.  The reference's CPU MATMUL! gives each (row, token) the decode product's bits
(batch.lisp:10-12); so do these kernels, so every comparison is bit for bit -- dense
(Q8_0, Q4_K, Q6_K) and the grouped expert product (IQ2_XXS, Q2_K) of a prefill chunk."""
import numpy as np
import pytest

import oracle_lib as orc
from illatio_amd import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    from illatio_amd import hip
    return hip.open_hip(0)


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


CASES = [
    (synth.Q8_0, 4864, 896, 70),        # the benchmark's config 1's matrices, a ragged token count
    (synth.Q8_0, 896, 4864, 5),
    (synth.Q8_0, 100, 64, 129),         # rows and columns that fill no tile
    (synth.Q4_K, 1024, 2560, 64),
    (synth.Q4_K, 200, 512, 3),
    (synth.Q6_K, 640, 5120, 96),        # the benchmark's config 3's format and width, fewer rows
    (synth.Q6_K, 65, 256, 65),
    (synth.Q6_K, 300, 1024, 333),       # three row tiles and three token tiles of 128, the last of each ragged
    (synth.Q6_K, 256, 768, 128),        # an odd number of super-blocks
    (synth.Q8_0, 300, 1024, 333),
    (synth.Q4_K, 300, 1024, 333),
    (synth.Q4_K, 256, 768, 128),
]


# ILT_I8_PLANES: "0" = the 64 x 64 kernel always, "1" = always the pipelined kernels (Q6_K and Q4_K as two int8 planes, Q8_0
# a block per MFMA), else only with enough tokens and rows to fill their 128 x 128 tiles.  The planes' kernel takes 64-row
# tiles where 128-row tiles would leave most CUs idle -- every shape here -- and ILT_I8P_TM=128 holds it to the large tile
# ("1/128").
@pytest.mark.parametrize("planes", [None, "0", "1", "1/128"])
@pytest.mark.parametrize("qtype,rows,cols,n", CASES)
def test_dense_prefill_equals_cpu_matmul_bit_for_bit(dev, monkeypatch, qtype, rows, cols, n, planes):
    from illatio_amd import dense, hip
    monkeypatch.delenv("ILT_I8P_TM", raising=False)
    if planes is None:
        monkeypatch.delenv("ILT_I8_PLANES", raising=False)
    elif cols % 64 or (planes == "1/128" and qtype == synth.Q8_0):
        pytest.skip("one kernel for this format")
    else:
        monkeypatch.setenv("ILT_I8_PLANES", planes[0])
        if planes == "1/128":
            monkeypatch.setenv("ILT_I8P_TM", "128")
    rng = synth.make_rng(qtype * 31 + rows + n)
    w = synth.weights(qtype, rows, cols, rng)
    x = synth.activations((n, cols), rng)
    x[0, :256] = 0.0
    bias = synth.activations(rows, rng)
    m = dense.upload_gmat(dev, "w", qtype, rows, cols, w)
    act = dense.QAct(dev, n, cols, ("q8",) if qtype == synth.Q8_0 else ("q8k",))
    xb, bb = hip.hip_upload_new(dev, x), hip.hip_upload_new(dev, bias)
    y = hip.hip_alloc(dev, 4 * n * rows)
    dense.quantize_act(dev, xb, act)
    dense.cmat_mul(dev, m, act, y, n=n)
    want = orc.matmul(qtype, w, rows, cols, x, nthreads=8)
    got = hip.hip_floats(y, n * rows).reshape(n, rows)
    assert np.array_equal(bits(got), bits(want)), (np.abs(got - want).max(), np.argwhere(bits(got) != bits(want))[:5])
    dense.cmat_mul(dev, m, act, y, n=n, bias=bb, acc=True)
    assert np.array_equal(bits(hip.hip_floats(y, n * rows).reshape(n, rows)), bits(want + (want + bias[None, :])))
    # the tiled product and the matrix-vector kernel agree on token 0
    y1 = hip.hip_alloc(dev, 4 * rows)
    dense.cmat_mul(dev, m, act, y1, n=1)
    assert np.array_equal(bits(hip.hip_floats(y1, rows)), bits(want[0]))
    for b in (xb, bb, y, y1):
        hip.hip_free(b)
    act.free(); m.free()


@pytest.mark.parametrize("rows,cols,n", [(640, 5120, 96), (65, 256, 65), (300, 1024, 333), (256, 768, 128)])
def test_two_pass_exact_product_bit_for_bit(dev, rows, cols, n):
    """The Q6_K product from planes written beforehand (planes_i8, mm_i8_planes): the planes hold
    scale * (quant - 32) + 4128 split into bytes, and the product is the CPU's, bias and
    accumulation included."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(rows + cols + n)
    w = synth.weights(synth.Q6_K, rows, cols, rng)
    x = synth.activations((n, cols), rng)
    x[0, :256] = 0.0
    bias = synth.activations(rows, rng)
    m = dense.upload_gmat(dev, "w", synth.Q6_K, rows, cols, w)
    act = dense.QAct(dev, n, cols, ("q8k",))
    xb, bb = hip.hip_upload_new(dev, x), hip.hip_upload_new(dev, bias)
    y = hip.hip_alloc(dev, 4 * n * rows)
    dense.quantize_act(dev, xb, act)
    planes = dense.planes_i8(dev, m)
    # every weight back from its planes: 256 * hi + (lo - 128 as a signed byte ... + 128) - 4128 = sc * (q - 32)
    nbytes = dense.planes_bytes(rows, cols)
    wh = dense.planes_to_rows(hip.hip_download(planes[0], np.uint8, nbytes), rows, cols).astype(np.int64).reshape(-1)
    wl = dense.planes_to_rows(hip.hip_download(planes[1], np.int8, nbytes), rows, cols).astype(np.int64).reshape(-1)
    deq = orc.dequant_rows(synth.Q6_K, w, cols).reshape(rows, cols // 256, 256)
    d = hip.hip_floats(planes[2], rows * (cols // 256)).reshape(rows, cols // 256)
    back = d[:, :, None] * (256 * wh + wl + 128 - 4128).reshape(rows, cols // 256, 256).astype(np.float32)
    assert np.array_equal(back, deq), (np.abs(back - deq).max(), np.argwhere(back != deq)[:5])      # (as numbers: a zero's sign may differ)
    dense.mat_mul_i8_planes(dev, planes, rows, cols, act, y, n)
    want = orc.matmul(synth.Q6_K, w, rows, cols, x, nthreads=8)
    got = hip.hip_floats(y, n * rows).reshape(n, rows)
    assert np.array_equal(bits(got), bits(want)), (np.abs(got - want).max(), np.argwhere(bits(got) != bits(want))[:5])
    dense.mat_mul_i8_planes(dev, planes, rows, cols, act, y, n, bias=bb, acc=True)
    assert np.array_equal(bits(hip.hip_floats(y, n * rows).reshape(n, rows)), bits(want + (want + bias[None, :])))
    for b in (xb, bb, y) + tuple(planes):
        hip.hip_free(b)
    act.free(); m.free()


def test_mm_q8_mma2_three_matrices_on_the_same_tokens(dev):
    """mm_q8_mma2 (dense.cu:884): Q, K and V of a prefill chunk in one call, each with mm_q8's (the
    CPU matmul!'s) bits; a matrix of no rows takes no part."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(515)
    cols, n = 896, 70
    shape = [896, 128, 136]
    ws = [synth.weights(synth.Q8_0, r, cols, rng) for r in shape]
    ms = [dense.upload_gmat(dev, f"w{i}", synth.Q8_0, r, cols, w) for i, (r, w) in enumerate(zip(shape, ws))]
    x = synth.activations((n, cols), rng)
    xb = hip.hip_upload_new(dev, x)
    act = dense.QAct(dev, n, cols, ("q8",))
    dense.quantize_act(dev, xb, act, n=n)
    bias = [synth.activations(r, rng) for r in shape]
    bbs = [hip.hip_upload_new(dev, b) for b in bias]
    ys = [hip.hip_alloc(dev, 4 * n * r) for r in shape]
    grid = ((n + 63) // 64, sum((r + 127) // 128 for r in shape))
    hip.launch(dev, "mm_q8_mma2", grid, 256, [ms[0].qs, ms[0].d, ys[0], bbs[0], shape[0], ms[1].qs, ms[1].d, ys[1], None, shape[1],
                                              ms[2].qs, ms[2].d, ys[2], bbs[2], shape[2], act.xq, act.xs, cols, n, 0])
    want = [np.stack([orc.matmul(synth.Q8_0, w, r, cols, x[t]) for t in range(n)]) for w, r in zip(ws, shape)]
    want[0] = want[0] + bias[0]; want[2] = want[2] + bias[2]
    for i, r in enumerate(shape):
        assert np.array_equal(bits(hip.hip_floats(ys[i], n * r)), bits(want[i].reshape(-1))), i
    # the middle matrix absent, the others accumulated onto what is there
    hip.launch(dev, "mm_q8_mma2", grid, 256, [ms[0].qs, ms[0].d, ys[0], None, shape[0], None, None, None, None, 0,
                                              ms[2].qs, ms[2].d, ys[2], None, shape[2], act.xq, act.xs, cols, n, 1])
    plain = [np.stack([orc.matmul(synth.Q8_0, w, r, cols, x[t]) for t in range(n)]) for w, r in zip(ws, shape)]
    assert np.array_equal(bits(hip.hip_floats(ys[0], n * shape[0])), bits((want[0] + plain[0]).reshape(-1)))
    assert np.array_equal(bits(hip.hip_floats(ys[1], n * shape[1])), bits(want[1].reshape(-1)))
    assert np.array_equal(bits(hip.hip_floats(ys[2], n * shape[2])), bits((want[2] + plain[2]).reshape(-1)))
    for b in [xb] + bbs + ys:
        hip.hip_free(b)
    act.free()
    for m in ms:
        m.free()


@pytest.mark.parametrize("qtype,n", [(synth.Q4_K, 200), (synth.Q6_K, 130), (synth.Q4_K, 40)])
def test_mm_k_n_matrices_on_the_same_tokens(dev, qtype, n):
    """mm_k_n: up to three K-quant matrices of one type on the same tokens, their row tiles in one launch (ragged row
    counts, one with a bias, the middle one absent, accumulation) -- each with the CPU matmul!'s bits, which are
    mm_k's; 40 tokens: too few for the shared launch, the call falls back on one product after another."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(616 + n)
    cols = 512
    shape = [300, 128, 520]
    ws = [synth.weights(qtype, r, cols, rng) for r in shape]
    ms = [dense.upload_gmat(dev, f"w{i}", qtype, r, cols, w) for i, (r, w) in enumerate(zip(shape, ws))]
    x = synth.activations((n, cols), rng)
    xb = hip.hip_upload_new(dev, x)
    act = dense.QAct(dev, n, cols, ("q8k",))
    dense.quantize_act(dev, xb, act, n=n)
    bias = synth.activations(shape[2], rng)
    bb = hip.hip_upload_new(dev, bias)
    ys = [hip.hip_alloc(dev, 4 * n * r) for r in shape]
    code = dense.KQUANT_CODE[qtype]
    grid = ((n + 127) // 128, sum((r + 127) // 128 for r in shape))
    tail = [act.kq, act.kd, act.ksum, cols, n]
    hip.launch(dev, "mm_k_n", grid, 512, [code, ms[0].qs, ys[0], None, shape[0], ms[1].qs, ys[1], None, shape[1],
                                          ms[2].qs, ys[2], bb, shape[2]] + tail + [0])
    plain = [orc.matmul(qtype, w, r, cols, x, nthreads=8).reshape(n, r) for w, r in zip(ws, shape)]
    want = [plain[0], plain[1], plain[2] + bias]
    for i, r in enumerate(shape):
        assert np.array_equal(bits(hip.hip_floats(ys[i], n * r)), bits(want[i].reshape(-1))), i
    # the middle matrix absent, the others accumulated onto what is there
    hip.launch(dev, "mm_k_n", grid, 512, [code, ms[0].qs, ys[0], None, shape[0], None, None, None, 0,
                                          ms[2].qs, ys[2], None, shape[2]] + tail + [1])
    assert np.array_equal(bits(hip.hip_floats(ys[0], n * shape[0])), bits((want[0] + plain[0]).reshape(-1)))
    assert np.array_equal(bits(hip.hip_floats(ys[1], n * shape[1])), bits(want[1].reshape(-1)))
    assert np.array_equal(bits(hip.hip_floats(ys[2], n * shape[2])), bits((want[2] + plain[2]).reshape(-1)))
    # the host's grouping: matrices of another type or width go on their own
    otype = synth.Q6_K if qtype == synth.Q4_K else synth.Q4_K
    ow = synth.weights(otype, 256, cols, rng)
    other = dense.upload_gmat(dev, "o", otype, 256, cols, ow)
    yo = hip.hip_alloc(dev, 4 * n * 256)
    dense.cmat_mul_n(dev, [(ms[0], ys[0], None), (other, yo, None), (ms[1], ys[1], None), (ms[2], ys[2], bb)], act, n)
    for i, r in enumerate(shape):
        assert np.array_equal(bits(hip.hip_floats(ys[i], n * r)), bits(want[i].reshape(-1))), i
    assert np.array_equal(bits(hip.hip_floats(yo, n * 256)), bits(orc.matmul(otype, ow, 256, cols, x, nthreads=8).reshape(-1)))
    for b in [xb, bb, yo] + ys:
        hip.hip_free(b)
    act.free()
    for m in ms + [other]:
        m.free()


def test_products_of_no_tokens_write_nothing(dev):
    """No tokens (an empty chunk): every prefill product returns without touching y."""
    from illatio_amd import dense, hip
    rows, cols = 256, 512
    rng = synth.make_rng(5)
    mark = synth.activations(4 * rows, rng)
    y = hip.hip_upload_new(dev, mark)
    for qtype in (synth.Q8_0, synth.Q4_K, synth.Q6_K):
        m = dense.upload_gmat(dev, "w", qtype, rows, cols, synth.weights(qtype, rows, cols, rng))
        act = dense.QAct(dev, 4, cols, ("q8",) if qtype == synth.Q8_0 else ("q8k",))
        dense.cmat_mul(dev, m, act, y, n=0)
        if qtype != synth.Q8_0:
            xb = hip.hip_alloc(dev, 2 * 4 * cols)
            dense.cmat_mul_bf16(dev, m, xb, y, 0)
            wb = dense.dequant_bf16(dev, m)
            dense.mat_mul_bf16(dev, wb, rows, cols, xb, y, 0)
            hip.hip_free(xb); hip.hip_free(wb)
        if qtype == synth.Q6_K:
            planes = dense.planes_i8(dev, m)
            dense.mat_mul_i8_planes(dev, planes, rows, cols, act, y, 0)
            for b in planes:
                hip.hip_free(b)
        act.free(); m.free()
    assert np.array_equal(bits(hip.hip_floats(y, 4 * rows)), bits(mark))
    hip.hip_free(y)


@pytest.mark.parametrize("ne,d,ff,nu,n,clamp", [(8, 512, 256, 3, 37, 0.0), (16, 1024, 512, 4, 150, 0.6),
                                                 (12, 4096, 2048, 6, 96, 0.0)])
@pytest.mark.parametrize("planes", [None, "0", "1"])        # the down product (Q2_K) on the 64 x 64 kernel / on the planes kernel
def test_moe_prefill_chunk_bit_exact(dev, monkeypatch, ne, d, ff, nu, n, clamp, planes):
    """the benchmark's config 5's sequence (route -> group -> gather -> grouped gate, up -> gated
    activation -> grouped down -> slot-ordered sum + shared) at reduced expert and token
    counts, Zipf-skewed routing, against the CPU path's chunk (ds4f.lisp:1169-1239)."""
    from illatio_amd import ds4f, hip
    if planes is None:
        monkeypatch.delenv("ILT_I8_PLANES", raising=False)
    else:
        monkeypatch.setenv("ILT_I8_PLANES", planes)
    rng = synth.make_rng(ne + d + n)
    gate = synth.weights(synth.IQ2_XXS, ne * ff, d, rng)
    up = synth.weights(synth.IQ2_XXS, ne * ff, d, rng)
    down = synth.weights(synth.Q2_K, ne * d, ff, rng)
    norms = synth.activations((n, d), rng)
    logits = synth.zipf_router_logits(n, ne, rng)
    shared = synth.activations((n, d), rng)
    want, wsel, ww, wcounts = orc.moe_chunk(gate, up, down, d, ff, ne, nu, 1.5, clamp, logits, norms, shared, nthreads=8)
    pool = ds4f.ExpertPool(dev, ne, d, ff, gate, up, down)
    lb, nb, sb = (hip.hip_upload_new(dev, a) for a in (logits, norms, shared))
    keep = {}
    moe = ds4f.ffn_routed_chunk(dev, pool, lb, nb, sb, n, ne, nu, 1.5, clamp, keep=keep)
    assert np.array_equal(keep["sel"], wsel.astype(np.uint32))
    assert np.array_equal(bits(keep["w"]), bits(ww))
    assert np.array_equal(keep["counts"], wcounts.astype(np.uint32))
    got = hip.hip_floats(moe, n * d).reshape(n, d)
    assert np.array_equal(bits(got), bits(want)), (np.abs(got - want).max(), np.argwhere(bits(got) != bits(want))[:5])
    for b in (lb, nb, sb, moe):
        hip.hip_free(b)
    pool.free()


@pytest.mark.parametrize("rows,cols,n", [(256, 4096, 70), (37, 48, 5), (300, 1024, 129)])
def test_d4_mm_f16_router_product_bit_exact(dev, rows, cols, n):
    """d4_mm_f16 (ds4f_mm.cu:253): an F16 matrix on float rows, every dot in F32-DOT16's order (the CPU's f32mm!,
    ds4f.lisp:278-293; the router's logits of a chunk), with the tokens' rows and the outputs strided."""
    from illatio_amd import ds4f, hip
    rng = synth.make_rng(rows + cols + n)
    w = (rng.standard_normal((rows, cols)) * 0.05).astype(np.float16)
    x = synth.activations((n, cols), rng)
    want = orc.f16mm(w.view(np.uint16), rows, cols, x)
    wb, xb = hip.hip_upload_new(dev, w.view(np.uint16)), hip.hip_upload_new(dev, x)
    y = hip.hip_alloc(dev, 4 * n * rows)
    ds4f.dk_mm(dev, "d4_mm_f16", wb, None, 2 * cols, rows, cols, xb, y, n)
    got = hip.hip_floats(y, n * rows).reshape(n, rows)
    assert np.array_equal(bits(got), bits(want)), np.abs(got - want).max()
    # strides: the tokens' rows and the outputs farther apart (cuda-ds4f-prefill.lisp:154 writes 32 apart)
    xs, ys = cols + 16, rows + 7
    xpad = np.zeros((n, xs), np.float32); xpad[:, :cols] = x
    xb2, y2 = hip.hip_upload_new(dev, xpad), hip.hip_alloc(dev, 4 * n * ys)
    ds4f.dk_mm(dev, "d4_mm_f16", wb, None, 2 * cols, rows, cols, xb2, y2, n, x_stride=xs, y_stride=ys)
    got2 = hip.hip_floats(y2, n * ys).reshape(n, ys)
    assert np.array_equal(bits(got2[:, :rows]), bits(want)) and not got2[:, rows:].any()
    for b in (wb, xb, y, xb2, y2):
        hip.hip_free(b)


@pytest.mark.parametrize("qtype,rows,cols,n", [(synth.Q8_0, 2048, 4096, 130), (synth.Q8_0, 100, 96, 7), (synth.Q2_K, 512, 2048, 200),
                                               (synth.IQ2_XXS, 300, 1024, 33), (synth.Q8_0, 4096, 2048, 1)])
def test_d4_mm_on_float_rows_bit_exact(dev, qtype, rows, cols, n):
    """d4_mm_q8_0 / d4_mm_q2_k / d4_mm_iq2_xxs (ds4f_mm.cu:252-255) take float rows; each token's result is the CPU
    path's: quantize-q8! with a float scale and the Q8_0 row dot (q8mv!, ds4f.lisp:294-297), or quantize-q8k! and
    the expert formats' row dots.  Two calls of different sizes in a row (the library's room for the quantized rows
    grows); strides shorter than a row are refused."""
    from illatio_amd import dense, ds4f, hip
    rng = synth.make_rng(qtype * 13 + rows + n)
    w = synth.weights(qtype, rows, cols, rng)
    name = {synth.Q8_0: "d4_mm_q8_0", synth.Q2_K: "d4_mm_q2_k", synth.IQ2_XXS: "d4_mm_iq2_xxs"}[qtype]
    if qtype == synth.Q8_0:
        m = dense.upload_gmat(dev, "w", qtype, rows, cols, w)
        wq, wd, rb = m.qs, m.d, 0
    else:
        wq, wd, rb = hip.hip_upload_new(dev, w), None, synth.row_bytes(qtype, cols)
    if qtype == synth.Q2_K:                                   # the library's room for the quantized rows sized beforehand
        import ctypes as C
        hip.call("ilt_d4_mm_reserve", C.c_int(n), C.c_int(cols))
    for ntok in (n, max(1, n // 3), n):
        x = synth.activations((ntok, cols), rng)
        x[0, :32] = 0.0
        xb, y = hip.hip_upload_new(dev, x), hip.hip_alloc(dev, 4 * ntok * rows)
        ds4f.dk_mm(dev, name, wq, wd, rb, rows, cols, xb, y, ntok)
        got = hip.hip_floats(y, ntok * rows).reshape(ntok, rows)
        want = orc.matmul(qtype, w, rows, cols, x, f16_scale=False, nthreads=8).reshape(ntok, rows)
        assert np.array_equal(bits(got), bits(want)), (ntok, np.abs(got - want).max())
        if ntok == n:
            with pytest.raises(hip.HipError):
                ds4f.dk_mm(dev, name, wq, wd, rb, rows, cols, xb, y, ntok, y_stride=rows - 1)
            with pytest.raises(hip.HipError):
                ds4f.dk_mm(dev, name, wq, wd, rb, rows, cols, xb, y, ntok, x_stride=cols - 4)
        hip.hip_free(xb); hip.hip_free(y)
    if qtype == synth.Q8_0:
        m.free()
    else:
        hip.hip_free(wq)


def test_d4_mm_on_two_streams_at_once(dev):
    """d4_mm_* calls queued on two streams of one GPU at once: each stream's calls quantize their rows into a buffer of
    that stream's (one sized beforehand through ilt_d4_mm_reserve_stream, the other grown by its first call), so both
    give what each gives alone."""
    import ctypes as C
    from illatio_amd import ds4f, hip
    info = hip.DeviceInfo()
    hip.call("ilt_device_get_info", C.c_int(dev.index), C.byref(info))
    other = hip.Device(dev.index, info, hip.hip_stream_create(dev))
    rng = synth.make_rng(131)
    rows, cols, n = 1024, 2048, 300
    rb = synth.row_bytes(synth.Q2_K, cols)
    hip.call("ilt_d4_mm_reserve_stream", C.c_uint64(other.stream), C.c_int(n), C.c_int(cols))
    sets = []
    for d_ in (dev, other):
        w = synth.weights(synth.Q2_K, rows, cols, rng)
        x = synth.activations((n, cols), rng)
        sets.append((d_, hip.hip_upload_new(d_, w), hip.hip_upload_new(d_, x), hip.hip_alloc(d_, 4 * n * rows),
                     orc.matmul(synth.Q2_K, w, rows, cols, x, nthreads=8).reshape(n, rows)))
    for _ in range(3):
        for d_, wq, xb, y, _w in sets:
            hip.hip_zero(y)
            for _ in range(6):
                ds4f.dk_mm(d_, "d4_mm_q2_k", wq, None, rb, rows, cols, xb, y, n)
        hip.hip_sync(dev); hip.hip_stream_sync(other.stream)
        for d_, wq, xb, y, want in sets:
            assert np.array_equal(bits(hip.hip_floats(y, n * rows).reshape(n, rows)), bits(want))
    for d_, wq, xb, y, _w in sets:
        for b in (wq, xb, y):
            hip.hip_free(b)


@pytest.mark.parametrize("groups,rank,gdim,n", [(4, 128, 512, 130), (3, 48, 96, 9), (8, 256, 1024, 257)])
def test_d4_mm_q8_0_grouped_attention_output_strided(dev, groups, rank, gdim, n):
    """The reference's strided call of d4_mm_q8_0 (cuda-ds4f-prefill.lisp:277-281): the grouped attention output
    product runs once a group on a slice of each token's heads (x_stride = nh*hd floats between tokens) with that
    group's rows of the matrix (the quants and the scales at offsets into their arrays), into a slice of each
    token's low row (y_stride = groups*rank).  Every (token, group) has the CPU path's bits: quantize-q8! with a
    float scale on the group's slice, the Q8_0 row dots of the group's rows."""
    from illatio_amd import dense, ds4f, hip
    rng = synth.make_rng(groups * 1000 + n)
    rows = groups * rank
    w = synth.weights(synth.Q8_0, rows, gdim, rng)
    m = dense.upload_gmat(dev, "attn_output_a", synth.Q8_0, rows, gdim, w)
    heads = synth.activations((n, groups * gdim), rng)
    hb = hip.hip_upload_new(dev, heads)
    low = hip.hip_alloc(dev, 4 * n * rows)
    hip.hip_zero(low)
    for g in range(groups):
        ds4f.dk_mm(dev, "d4_mm_q8_0", m.qs.at(g * rank * gdim), m.d.at(2 * g * rank * (gdim // 32)), 0, rank, gdim,
                   hb.at(4 * g * gdim), low.at(4 * g * rank), n, x_stride=groups * gdim, y_stride=rows)
    got = hip.hip_floats(low, n * rows).reshape(n, groups, rank)
    for g in range(groups):
        xg = np.ascontiguousarray(heads[:, g * gdim:(g + 1) * gdim])
        wg = np.ascontiguousarray(w[g * rank:(g + 1) * rank])
        want = orc.matmul(synth.Q8_0, wg, rank, gdim, xg, f16_scale=False, nthreads=8).reshape(n, rank)
        assert np.array_equal(bits(got[:, g]), bits(want)), (g, np.abs(got[:, g] - want).max())
    hip.hip_free(hb); hip.hip_free(low); m.free()


@pytest.mark.parametrize("qtype,rows,cols,n", [(synth.Q2_K, 256, 512, 140), (synth.IQ2_XXS, 70, 256, 5)])
def test_d4_mm_k_formats_strided(dev, qtype, rows, cols, n):
    """d4_mm_q2_k / d4_mm_iq2_xxs with the tokens' rows and results further apart than their widths: what lies between
    is neither read nor written."""
    from illatio_amd import ds4f, hip
    rng = synth.make_rng(qtype + rows + n)
    w = synth.weights(qtype, rows, cols, rng)
    name = {synth.Q2_K: "d4_mm_q2_k", synth.IQ2_XXS: "d4_mm_iq2_xxs"}[qtype]
    wb = hip.hip_upload_new(dev, w)
    xs, ys = cols + 64, rows + 24
    x = synth.activations((n, xs), rng)
    x[:, cols:] = np.nan
    xb, y = hip.hip_upload_new(dev, x), hip.hip_upload_new(dev, np.full((n, ys), 7.0, np.float32))
    ds4f.dk_mm(dev, name, wb, None, synth.row_bytes(qtype, cols), rows, cols, xb, y, n, x_stride=xs, y_stride=ys)
    got = hip.hip_floats(y, n * ys).reshape(n, ys)
    want = orc.matmul(qtype, w, rows, cols, np.ascontiguousarray(x[:, :cols]), nthreads=8).reshape(n, rows)
    assert np.array_equal(bits(got[:, :rows]), bits(want))
    assert (got[:, rows:] == 7.0).all()
    for b in (wb, xb, y):
        hip.hip_free(b)
