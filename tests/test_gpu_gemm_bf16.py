"""GPU checks of the bf16 matrix-core prefill products, through the C ABI.

Two kinds.  (1) One-hot activations read the dequantized matrix back through the product:
token t = column c's unit vector gives y[t][r] = bf16(W[r][c]) with nothing else added, so
every weight's position, scale and sign is compared exactly with the CPU dequantizer's
value rounded to bf16.  (2) Random activations against the CPU path (quantized activations,
integer block dots) and against a double-precision product of the dequantized weights with
the float activations.  The tolerance of this path is 2e-2 of the largest output magnitude
against the CPU path; against the double product the bf16 roundings alone remain, and the
rms error must stay under 5e-3 of the rms output."""
import numpy as np
import pytest

import oracle_lib as orc
from illatio_amd import synth

pytestmark = pytest.mark.gpu

TOL_VS_CPU = 2e-2      # max |gpu - cpu| / max |cpu|
TOL_RMS_VS_EXACT = 5e-3
TOL_CHAIN_VS_EXACT = 2e-2   # the whole chain (three products, a clamped gate) against the exact double-precision chain


@pytest.fixture(scope="module")
def dev():
    from illatio_amd import hip
    return hip.open_hip(0)


def bf16_round(a):
    """float32 -> nearest bf16 (ties to even), returned as float32."""
    b = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    b = (b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000
    return b.astype(np.uint32).view(np.float32)


def upload(dev, qtype, rows, cols, w):
    from illatio_amd import dense, hip
    if qtype in (synth.Q4_K, synth.Q6_K):
        return dense.upload_gmat(dev, "w", qtype, rows, cols, w)
    return dense.CMat("w", qtype, rows, cols, hip.hip_upload_new(dev, w))


FORMATS = [synth.Q4_K, synth.Q6_K, synth.Q2_K, synth.IQ2_XXS]


@pytest.mark.parametrize("tile", [1, 2, 3])       # the 128x128, 128x256 and 256x256 tiles
@pytest.mark.parametrize("qtype", FORMATS)
@pytest.mark.parametrize("rows,cols", [(130, 512), (300, 256)])
def test_one_hot_tokens_read_back_the_dequantized_matrix(dev, monkeypatch, qtype, rows, cols, tile):
    from illatio_amd import dense, hip
    monkeypatch.setenv("ILT_BF16_TILE", str(tile))
    rng = synth.make_rng(qtype + rows)
    w = synth.weights(qtype, rows, cols, rng)
    x = np.eye(cols, dtype=np.float32)
    m = upload(dev, qtype, rows, cols, w)
    xf, y = hip.hip_upload_new(dev, x), hip.hip_alloc(dev, 4 * cols * rows)
    xb = dense.cvt_bf16(dev, xf, x.size)
    dense.cmat_mul_bf16(dev, m, xb, y, cols)
    got = hip.hip_floats(y, cols * rows).reshape(cols, rows)
    want = bf16_round(orc.dequant_rows(qtype, w, cols).reshape(rows, cols)).T
    # compared as numbers: a weight that dequantizes to -0.0 comes back as 0.0 + -0.0 = 0.0
    assert np.array_equal(got, want), np.argwhere(got != want)[:8]
    hip.hip_free(xf); hip.hip_free(xb); hip.hip_free(y); m.free()


@pytest.mark.parametrize("qtype,rows,cols,n", [
    (synth.Q6_K, 640, 5120, 200),        # the benchmark's config 3's format and width, fewer rows, ragged tokens
    (synth.Q6_K, 1000, 1024, 128),
    (synth.Q4_K, 1024, 2560, 77),
    (synth.Q2_K, 300, 2048, 129),
    (synth.IQ2_XXS, 256, 4096, 64),
    (synth.Q6_K, 8200, 512, 4000),       # enough tiles that the largest tile is chosen by itself; ragged both ways
])
@pytest.mark.parametrize("tile", [0, 1, 2, 3])       # 0: chosen by shape; others: that tile forced
def test_dense_bf16_product_within_tolerance(dev, monkeypatch, qtype, rows, cols, n, tile):
    from illatio_amd import dense, hip
    if tile:
        monkeypatch.setenv("ILT_BF16_TILE", str(tile))
    else:
        monkeypatch.delenv("ILT_BF16_TILE", raising=False)
    rng = synth.make_rng(qtype * 7 + rows + n)
    w = synth.weights(qtype, rows, cols, rng)
    x = synth.activations((n, cols), rng)
    bias = synth.activations(rows, rng)
    m = upload(dev, qtype, rows, cols, w)
    xf, bb, y = hip.hip_upload_new(dev, x), hip.hip_upload_new(dev, bias), hip.hip_alloc(dev, 4 * n * rows)
    xb = dense.cvt_bf16(dev, xf, x.size)
    assert np.array_equal(hip.hip_download(xb, np.uint16, x.size), (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16).ravel())
    dense.cmat_mul_bf16(dev, m, xb, y, n)
    got = hip.hip_floats(y, n * rows).reshape(n, rows)
    cpu = orc.matmul(qtype, w, rows, cols, x, nthreads=16)
    exact = x.astype(np.float64) @ orc.dequant_rows(qtype, w, cols).reshape(rows, cols).astype(np.float64).T
    assert np.abs(got - cpu).max() <= TOL_VS_CPU * np.abs(cpu).max()
    assert np.sqrt(np.mean((got - exact) ** 2)) <= TOL_RMS_VS_EXACT * np.sqrt(np.mean(exact ** 2))
    # accumulate + bias: y += W x + bias
    dense.cmat_mul_bf16(dev, m, xb, y, n, bias=bb, acc=True)
    got2 = hip.hip_floats(y, n * rows).reshape(n, rows)
    assert np.array_equal(got2, got + (got + bias[None, :]))
    for b in (xf, xb, bb, y):
        hip.hip_free(b)
    m.free()


@pytest.mark.parametrize("qtype,rows,cols,n,tile", [
    (synth.Q6_K, 8704, 2048, 512, 1),      # 272 tiles of 128 x 128: a whole round over the CUs, and 16 tiles split eight ways
    (synth.Q6_K, 4352, 2048, 500, 2),      # 68 tiles of 128 x 256, all split; ragged tokens
    (synth.Q4_K, 2560, 9728, 512, 0),      # a decoder's down product on a prompt's chunk: few tiles, many columns, 38 super-blocks split unevenly
    (synth.Q2_K, 700, 2048, 130, 0),       # ragged rows and tokens
])
def test_tiles_split_over_the_columns(dev, monkeypatch, qtype, rows, cols, n, tile):
    """Where a product's tiles do not fill a round over the CUs, the tiles of the last round are split over the columns'
    super-blocks and their parts added by a second kernel: the same product as unsplit but for the order of fp32 sums
    (within 1e-5 of the largest output), within the path's tolerance of the CPU path on a sample of the tokens, and
    bias and accumulation as the unsplit store applies them."""
    from illatio_amd import dense, hip
    if tile:
        monkeypatch.setenv("ILT_BF16_TILE", str(tile))
    else:
        monkeypatch.delenv("ILT_BF16_TILE", raising=False)
    rng = synth.make_rng(qtype * 13 + rows + n)
    w = synth.weights(qtype, rows, cols, rng)
    x = synth.activations((n, cols), rng)
    bias = synth.activations(rows, rng)
    m = upload(dev, qtype, rows, cols, w)
    xf, bb = hip.hip_upload_new(dev, x), hip.hip_upload_new(dev, bias)
    xb = dense.cvt_bf16(dev, xf, x.size)
    out = {}
    for split in ("0", None):
        if split is None:
            monkeypatch.delenv("ILT_BF16_SPLITK", raising=False)
        else:
            monkeypatch.setenv("ILT_BF16_SPLITK", split)
        y = hip.hip_upload_new(dev, np.full(n * rows + 64, 3.0, np.float32))
        dense.cmat_mul_bf16(dev, m, xb, y, n)
        a = hip.hip_floats(y, n * rows + 64)
        assert np.all(a[n * rows:] == 3.0)                       # nothing past the last token's rows
        dense.cmat_mul_bf16(dev, m, xb, y, n, bias=bb, acc=True)
        b = hip.hip_floats(y, n * rows).reshape(n, rows)
        a = a[:n * rows].reshape(n, rows)
        assert np.array_equal(b, a + (a + bias[None, :]))
        out[split] = a
        hip.hip_free(y)
    assert np.abs(out[None] - out["0"]).max() <= 1e-5 * np.abs(out["0"]).max()
    assert not np.array_equal(out[None], out["0"])               # (the split was taken: the sums' order shows somewhere)
    pick = np.unique(np.concatenate([np.arange(0, n, 37), [n - 1]]))
    cpu = orc.matmul(qtype, w, rows, cols, x[pick], nthreads=16)
    assert np.abs(out[None][pick] - cpu).max() <= TOL_VS_CPU * np.abs(cpu).max()
    for b_ in (xf, xb, bb):
        hip.hip_free(b_)
    m.free()


def test_split_products_on_two_streams_keep_their_parts_apart(dev):
    """Two split products queued on two streams of one GPU at once: each stream's launches keep their parts in a
    buffer of that stream's, so both give what each gives alone."""
    import ctypes as C
    from illatio_amd import dense, hip
    info = hip.DeviceInfo()
    hip.call("ilt_device_get_info", C.c_int(dev.index), C.byref(info))
    other = hip.Device(dev.index, info, hip.hip_stream_create(dev))
    rng = synth.make_rng(97)
    rows, cols, n = 2560, 9728, 512                           # 80 tiles of 128 x 128 or fewer of the larger: split either way
    ms, xs, ys, alone = [], [], [], []
    for d_ in (dev, other):
        w = synth.weights(synth.Q4_K, rows, cols, rng)
        x = synth.activations((n, cols), rng)
        m = upload(d_, synth.Q4_K, rows, cols, w)
        xf = hip.hip_upload_new(d_, x)
        xb = dense.cvt_bf16(d_, xf, x.size)
        y = hip.hip_alloc(d_, 4 * n * rows)
        dense.cmat_mul_bf16(d_, m, xb, y, n)
        alone.append(hip.hip_floats(y, n * rows))             # (waits for the stream)
        hip.hip_free(xf)
        ms.append(m); xs.append(xb); ys.append(y)
    for _ in range(3):                                         # both streams busy with split products at the same time
        for d_, m, xb, y in zip((dev, other), ms, xs, ys):
            hip.hip_zero(y)
            for _ in range(4):
                dense.cmat_mul_bf16(d_, m, xb, y, n)
        hip.hip_sync(dev); hip.hip_stream_sync(other.stream)
        for y, a in zip(ys, alone):
            assert np.array_equal(bits_of(hip.hip_floats(y, n * rows)), bits_of(a))
    for b_ in xs + ys:
        hip.hip_free(b_)
    for m in ms:
        m.free()


def bits_of(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("two_pass", [False, True])
def test_output_head_keeps_the_cpu_paths_top_token(dev, two_pass):
    """128 positions through an output head (Q6_K, config 2's width, 8192 of its rows): the
    bf16 product picks the CPU path's token at every position, except where the CPU path's
    own two best logits lie closer than 5 % of the position's logit spread -- the near-tie
    rule of the reference's consistency checks (cuda-consistency-test.lisp:20-22,
    vectors-test.lisp:26-27); the two paths' difference between two logits has an rms of
    1.6 % of the spread, most of it the CPU path's quantized activations -- and at 90 % of
    the positions at least (ds4f-vectors-test.lisp:30-32)."""
    from illatio_amd import dense, hip
    rows, cols, n = 8192, 2560, 128
    rng = synth.make_rng(4242)
    w = synth.weights(synth.Q6_K, rows, cols, rng)
    x = synth.activations((n, cols), rng)
    m = upload(dev, synth.Q6_K, rows, cols, w)
    xf, y = hip.hip_upload_new(dev, x), hip.hip_alloc(dev, 4 * n * rows)
    if two_pass:
        wb = dense.dequant_bf16(dev, m)
        xs = dense.cvt_bf16_slabs(dev, xf, n, cols)
        dense.mat_mul_bf16(dev, wb, rows, cols, xs, y, n)
        tmp = (wb, xs)
    else:
        xb = dense.cvt_bf16(dev, xf, x.size)
        dense.cmat_mul_bf16(dev, m, xb, y, n)
        tmp = (xb,)
    got = hip.hip_floats(y, n * rows).reshape(n, rows)
    cpu = orc.matmul(synth.Q6_K, w, rows, cols, x, nthreads=16)
    top, mine = cpu.argmax(1), got.argmax(1)
    best2 = np.sort(cpu, axis=1)[:, -2:]
    near_tie = (best2[:, 1] - best2[:, 0]) < 0.05 * cpu.std(axis=1)
    differ = top != mine
    assert not np.any(differ & ~near_tie), (np.argwhere(differ & ~near_tie).ravel(), near_tie.sum())
    assert differ.sum() <= n // 10, differ.sum()
    for b in (xf, y) + tmp:
        hip.hip_free(b)
    m.free()


def exact_chunk(G, U, Dn, sel, ww, norms, clamp):
    """The routed experts of a chunk in double precision from the dequantized weights and
    the float activations (no activation quantization, no bf16): what both paths approximate."""
    n, nu = sel.shape
    out = np.zeros((n, Dn.shape[1]))
    for t in range(n):
        x = norms[t].astype(np.float64)
        for s in range(nu):
            e = int(sel[t, s])
            g, u = G[e] @ x, U[e] @ x
            if clamp > 0:
                g, u = np.minimum(g, clamp), np.clip(u, -clamp, clamp)
            out[t] += Dn[e] @ ((g / (1 + np.exp(-g))) * u * float(ww[t, s]))
    return out


@pytest.mark.parametrize("ne,d,ff,nu,n,clamp", [(8, 512, 256, 3, 37, 0.0), (16, 1024, 512, 4, 300, 0.6),
                                                 (12, 4096, 2048, 6, 96, 0.0)])
# the default (256 x 128 tiles with the weights dequantized into registers where the rows allow), 128 x 128 always,
# 256 x 128 through LDS
@pytest.mark.parametrize("id_tile", [None, "1", "2"])
def test_moe_prefill_chunk_bf16_within_tolerance(dev, monkeypatch, ne, d, ff, nu, n, clamp, id_tile):
    """The prefill chunk of test_gpu_gemm.py with the three grouped products on the bf16
    matrix cores.  Routing, counts and weights stay equal to the CPU path's.  Each grouped
    product is within 2e-2 of the CPU product (quantized activations, integer block dots)
    of the same input rows.  Over the whole chain the CPU path's own activation quantization
    is the larger error (2-7% of the largest output at these shapes, against an exact
    double-precision chain), so the chain is held to this: the bf16 chunk is no farther
    from the exact chain than the CPU path's chunk is."""
    if id_tile is None:
        monkeypatch.delenv("ILT_BF16_ID_TILE", raising=False)
    else:
        monkeypatch.setenv("ILT_BF16_ID_TILE", id_tile)
    from illatio_amd import ds4f, hip
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
    moe = ds4f.ffn_routed_chunk_bf16(dev, pool, lb, nb, sb, n, ne, nu, 1.5, clamp, keep=keep)
    assert np.array_equal(keep["sel"], wsel.astype(np.uint32))
    assert np.array_equal(keep["w"].view(np.uint32), np.ascontiguousarray(ww, np.float32).view(np.uint32))
    assert np.array_equal(keep["counts"], wcounts.astype(np.uint32))
    got = hip.hip_floats(moe, n * d).reshape(n, d)

    # every expert's three products against the CPU product of the same rows
    grb, drb = synth.row_bytes(synth.IQ2_XXS, d), synth.row_bytes(synth.Q2_K, ff)
    gate_e, up_e, down_e = gate.reshape(ne, ff * grb), up.reshape(ne, ff * grb), down.reshape(ne, d * drb)
    cpu = {k: np.zeros_like(keep[k]) for k in ("gate", "up", "down")}
    for e in range(ne):
        b, c = int(keep["bases"][e]), int(keep["counts"][e])
        if c == 0:
            continue
        xrows = norms[keep["rmap"][b:b + c]]              # the rows the expert's tiles read through the row map
        cpu["gate"][b:b + c] = orc.matmul(synth.IQ2_XXS, gate_e[e], ff, d, xrows, nthreads=8)
        cpu["up"][b:b + c] = orc.matmul(synth.IQ2_XXS, up_e[e], ff, d, xrows, nthreads=8)
        cpu["down"][b:b + c] = orc.matmul(synth.Q2_K, down_e[e], d, ff, keep["mid"][b:b + c], nthreads=8)
    for k in ("gate", "up", "down"):
        assert np.abs(keep[k] - cpu[k]).max() <= TOL_VS_CPU * np.abs(cpu[k]).max(), k

    # the chain against the exact one
    G = orc.dequant_rows(synth.IQ2_XXS, gate, d).reshape(ne, ff, d).astype(np.float64)
    U = orc.dequant_rows(synth.IQ2_XXS, up, d).reshape(ne, ff, d).astype(np.float64)
    Dn = orc.dequant_rows(synth.Q2_K, down, ff).reshape(ne, d, ff).astype(np.float64)
    exact = exact_chunk(G, U, Dn, wsel, ww, norms, clamp) + shared
    err_gpu, err_cpu = np.abs(got - exact).max(), np.abs(want - exact).max()
    assert err_gpu <= err_cpu, (err_gpu, err_cpu)
    assert err_gpu <= TOL_CHAIN_VS_EXACT * np.abs(exact - shared).max(), (err_gpu, np.abs(exact - shared).max())
    for b in (lb, nb, sb, moe):
        hip.hip_free(b)
    pool.free()


@pytest.mark.parametrize("qtype,rows,cols,n", [
    (synth.Q6_K, 640, 5120, 200),
    (synth.Q4_K, 300, 256, 77),          # one ragged tile, two steps... and a single super-block of columns
    (synth.Q2_K, 513, 1024, 300),
    (synth.IQ2_XXS, 256, 4096, 256),
    (synth.Q6_K, 8200, 512, 4000),       # many tiles, ragged both ways
])
@pytest.mark.parametrize("split", [None, "0", "128"])      # tiles chosen by shape (256-tiles + 128-tiles for the rows left over), 256 only, 128 only
def test_two_pass_bf16_product(dev, monkeypatch, qtype, rows, cols, n, split):
    """dequant_bf16 writes each weight as the one-pass kernel rounds it; mm_bf16 on that copy adds
    the same products in the same order, so it returns the one-pass kernel's numbers (the one-pass kernel
    with its tiles whole: split over the columns it adds a tile's parts in another order)."""
    from illatio_amd import dense, hip
    monkeypatch.delenv("ILT_BF16_TILE", raising=False)
    monkeypatch.setenv("ILT_BF16_SPLITK", "0")
    if split is None:
        monkeypatch.delenv("ILT_BF16_PLAIN_SPLIT", raising=False)
    else:
        monkeypatch.setenv("ILT_BF16_PLAIN_SPLIT", split)
    rng = synth.make_rng(qtype * 11 + rows + n)
    w = synth.weights(qtype, rows, cols, rng)
    x = synth.activations((n, cols), rng)
    bias = synth.activations(rows, rng)
    m = upload(dev, qtype, rows, cols, w)
    wb = dense.dequant_bf16(dev, m)
    slabs = hip.hip_download(wb, np.uint16, dense.slabs_bytes(rows, cols) // 2)
    got_w = (dense.slabs_to_rows(slabs, rows, cols).astype(np.uint32) << 16).view(np.float32)
    want_w = bf16_round(orc.dequant_rows(qtype, w, cols)).reshape(rows, cols)
    assert np.array_equal(got_w, want_w), np.argwhere(got_w != want_w)[:8]       # as numbers: -0.0 == 0.0
    assert not dense.slabs_to_rows(slabs, (rows + 255) // 256 * 256, cols)[rows:].any()      # the padding rows are zeros
    xf, bb = hip.hip_upload_new(dev, x), hip.hip_upload_new(dev, bias)
    y1, y2 = hip.hip_alloc(dev, 4 * n * rows), hip.hip_alloc(dev, 4 * n * rows)
    xb = dense.cvt_bf16(dev, xf, x.size)
    xs = dense.cvt_bf16_slabs(dev, xf, n, cols)
    assert np.array_equal(dense.slabs_to_rows(hip.hip_download(xs, np.uint16, dense.slabs_bytes(n, cols) // 2), n, cols),
                          hip.hip_download(xb, np.uint16, x.size).reshape(n, cols))
    dense.cmat_mul_bf16(dev, m, xb, y1, n)
    dense.mat_mul_bf16(dev, wb, rows, cols, xs, y2, n)
    one = hip.hip_floats(y1, n * rows).reshape(n, rows)
    two = hip.hip_floats(y2, n * rows).reshape(n, rows)
    assert np.array_equal(one, two), np.argwhere(one != two)[:8]
    cpu = orc.matmul(qtype, w, rows, cols, x, nthreads=16)
    assert np.abs(two - cpu).max() <= TOL_VS_CPU * np.abs(cpu).max()
    dense.mat_mul_bf16(dev, wb, rows, cols, xs, y2, n, bias=bb, acc=True)
    assert np.array_equal(hip.hip_floats(y2, n * rows).reshape(n, rows), two + (two + bias[None, :]))
    dense.mat_mul_bf16(dev, wb, rows, cols, xs, y2, n, acc=True)                 # each of the four store loops
    assert np.array_equal(hip.hip_floats(y2, n * rows).reshape(n, rows), (two + (two + bias[None, :])) + two)
    dense.mat_mul_bf16(dev, wb, rows, cols, xs, y2, n, bias=bb)
    assert np.array_equal(hip.hip_floats(y2, n * rows).reshape(n, rows), two + bias[None, :])
    for b in (xf, xb, xs, bb, y1, y2, wb):
        hip.hip_free(b)
    m.free()


@pytest.mark.parametrize("ne,d,ff,nu,n,clamp", [(8, 512, 256, 3, 37, 0.0), (16, 1024, 512, 4, 300, 0.6), (4, 1024, 256, 2, 333, 0.0),
                                                 (6, 768, 256, 2, 70, 0.0)])      # the last: three super-blocks, three row tiles
def test_grouped_product_variants_agree_bitwise(dev, monkeypatch, ne, d, ff, nu, n, clamp):
    """The grouped product's variants make the same bf16 operands and add the same MFMA results
    in the same order, so their outputs are equal bit for bit: groups of a few rows (token
    patches skipped), of more than one tile of 128, and empty ones."""
    from illatio_amd import ds4f, hip
    rng = synth.make_rng(7 * ne + d + n)
    gate = synth.weights(synth.IQ2_XXS, ne * ff, d, rng)
    up = synth.weights(synth.IQ2_XXS, ne * ff, d, rng)
    down = synth.weights(synth.Q2_K, ne * d, ff, rng)
    norms = synth.activations((n, d), rng)
    logits = synth.zipf_router_logits(n, ne, rng)
    logits[:, ne - 1] = -30.0                             # an expert nobody picks
    shared = synth.activations((n, d), rng)
    pool = ds4f.ExpertPool(dev, ne, d, ff, gate, up, down)
    lb, nb, sb = (hip.hip_upload_new(dev, a) for a in (logits, norms, shared))
    res = {}
    for tile in (None, "1", "2"):
        if tile is None:
            monkeypatch.delenv("ILT_BF16_ID_TILE", raising=False)
        else:
            monkeypatch.setenv("ILT_BF16_ID_TILE", tile)
        keep = {}
        moe = ds4f.ffn_routed_chunk_bf16(dev, pool, lb, nb, sb, n, ne, nu, 1.5, clamp, keep=keep)
        keep["out"] = hip.hip_floats(moe, n * d)
        hip.hip_free(moe)
        # a group's rows in the order of their tokens (the scatter's order within a group varies from run to run)
        order = np.concatenate([int(b) + np.argsort(keep["rmap"][int(b):int(b) + int(c)], kind="stable")
                                for b, c in zip(keep["bases"], keep["counts"])])
        for k in ("gate", "up", "down"):
            keep[k] = keep[k][order]
        res[tile] = keep
    assert int(res[None]["counts"][ne - 1]) == 0 and int(res[None]["counts"].max()) > (128 if n >= 300 else 0)
    for tile in ("1", "2"):
        for k in ("gate", "up", "down", "out"):
            assert np.array_equal(res[None][k].view(np.uint32), res[tile][k].view(np.uint32)), (tile, k)
    # gate, up and the gated activation in one launch: the same bits again
    monkeypatch.delenv("ILT_BF16_ID_TILE", raising=False)
    keep = {}
    moe = ds4f.ffn_routed_chunk_bf16(dev, pool, lb, nb, sb, n, ne, nu, 1.5, clamp, keep=keep, fused=True)
    out = hip.hip_floats(moe, n * d)
    hip.hip_free(moe)
    assert "gate" not in keep
    order = np.concatenate([int(b) + np.argsort(keep["rmap"][int(b):int(b) + int(c)], kind="stable")
                            for b, c in zip(keep["bases"], keep["counts"])])
    order0 = np.concatenate([int(b) + np.argsort(res[None]["rmap"][int(b):int(b) + int(c)], kind="stable")
                             for b, c in zip(res[None]["bases"], res[None]["counts"])])
    assert np.array_equal(keep["mid"][order].view(np.uint32), res[None]["mid"][order0].view(np.uint32))
    assert np.array_equal(keep["down"][order].view(np.uint32), res[None]["down"].view(np.uint32))
    assert np.array_equal(out.view(np.uint32), res[None]["out"].view(np.uint32))
    for b in (lb, nb, sb):
        hip.hip_free(b)
    pool.free()
