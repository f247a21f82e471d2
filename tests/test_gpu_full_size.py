"""The products at the full sizes the benchmark configurations name, checked where the CPU oracle
would take minutes for everything through what the path itself guarantees: a prefill product's
token is that token's decode product (batch.lisp:10-12), so a sample of tokens (the first, the
last, tile edges) is compared with the oracle's row dots bit for bit; a chunk's token is that
token's own decode step (ds4f.lisp:1128-1130)."""
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


def test_output_head_of_config_2_bit_exact(dev):
    """The Q6_K output head, 151936 x 2560 (319 MB), on float activations with the norm inside the
    launch: every logit has the oracle's bits and the greedy token is the CPU path's."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(2024)
    rows, cols = 151936, 2560
    w = synth.weights(synth.Q6_K, rows, cols, rng)
    m = dense.upload_gmat(dev, "output", synth.Q6_K, rows, cols, w)
    nw = (synth.activations(cols, rng) * 0.2 + 1.0).astype(np.float32)
    nwb = hip.hip_upload_new(dev, nw)
    y = hip.hip_alloc(dev, 4 * rows)
    for trial in range(2):
        x = synth.activations(cols, rng)
        xb = hip.hip_upload_new(dev, x)
        dense.mv_multi(dev, [(m, y, None)], xf=xb, norm=(nwb, 1e-6))
        got = hip.hip_floats(y, rows)
        want = orc.matmul(synth.Q6_K, w, rows, cols, orc.rmsnorm(x, nw, 1e-6), nthreads=8).reshape(-1)
        assert np.array_equal(bits(got), bits(want)), np.argwhere(bits(got) != bits(want))[:5]
        assert int(np.argmax(got)) == int(np.argmax(want))
        hip.hip_free(xb)
    hip.hip_free(y); hip.hip_free(nwb)
    m.free()


@pytest.mark.parametrize("rows,cols", [(17408, 5120), (5120, 17408)])
def test_prefill_of_config_3_at_4096_tokens(dev, rows, cols):
    """Q6_K at the 27B-style shape on 4096 tokens: the exact product (from the quantized matrix and
    from the int8 planes) has the oracle's bits on the sampled tokens, and both give the same
    numbers for every token; the bf16 product is within 2e-2 of the CPU path on them."""
    from illatio_amd import dense, hip
    rng = synth.make_rng(rows + 7)
    T = 4096
    w = synth.weights(synth.Q6_K, rows, cols, rng, dscale=0.01)
    x = synth.activations((T, cols), rng)
    x[5, :512] = 0.0
    sample = [0, 1, 5, 127, 128, 255, 256, 2047, 2048, 4094, 4095]
    want = orc.matmul(synth.Q6_K, w, rows, cols, x[sample], nthreads=8)
    m = dense.upload_gmat(dev, "w", synth.Q6_K, rows, cols, w)
    xb = hip.hip_upload_new(dev, x)
    act = dense.QAct(dev, T, cols, ("q8k",))
    dense.quantize_act(dev, xb, act)
    y = hip.hip_alloc(dev, 4 * T * rows)
    dense.cmat_mul(dev, m, act, y, n=T)
    exact = hip.hip_floats(y, T * rows).reshape(T, rows)
    assert np.array_equal(bits(exact[sample]), bits(want))
    planes = dense.planes_i8(dev, m)
    hip.hip_zero(y)
    dense.mat_mul_i8_planes(dev, planes, rows, cols, act, y, T)
    two_pass = hip.hip_floats(y, T * rows).reshape(T, rows)
    assert np.array_equal(bits(two_pass), bits(exact))
    del two_pass
    for b in planes:
        hip.hip_free(b)
    # bf16, two passes
    wb = dense.dequant_bf16(dev, m)
    xs = dense.cvt_bf16_slabs(dev, xb, T, cols)
    dense.mat_mul_bf16(dev, wb, rows, cols, xs, y, T)
    got = hip.hip_floats(y, T * rows).reshape(T, rows)[sample]
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err <= 2e-2, err          # the tolerance the bf16 path is held to against the CPU path
    for b in (wb, xs, xb, y):
        hip.hip_free(b)
    act.free(); m.free()


@pytest.mark.parametrize("T", [512, 2048])
def test_prefill_of_config_3_at_512_and_2048_tokens(dev, T):
    """The 17408 x 5120 Q6_K matrix on 512 and on 2048 tokens, the sizes at which the host picks
    the one-pass kernels (weights dequantized inside the loop): the exact product has the oracle's
    bits on the sampled tokens, the bf16 product is within 2e-2 of the CPU path on them."""
    from illatio_amd import dense, hip
    rows, cols = 17408, 5120
    rng = synth.make_rng(rows + T)
    w = synth.weights(synth.Q6_K, rows, cols, rng, dscale=0.01)
    x = synth.activations((T, cols), rng)
    x[3, 256:1024] = 0.0
    sample = [0, 3, 127, 128, 255, 256, T // 2 - 1, T // 2, T - 2, T - 1]
    want = orc.matmul(synth.Q6_K, w, rows, cols, x[sample], nthreads=8)
    m = dense.upload_gmat(dev, "w", synth.Q6_K, rows, cols, w)
    xb = hip.hip_upload_new(dev, x)
    act = dense.QAct(dev, T, cols, ("q8k",))
    dense.quantize_act(dev, xb, act)
    y = hip.hip_alloc(dev, 4 * T * rows)
    dense.cmat_mul(dev, m, act, y, n=T)
    exact = hip.hip_floats(y, T * rows).reshape(T, rows)[sample]
    assert np.array_equal(bits(exact), bits(want))
    hip.hip_zero(y)
    xh = dense.cvt_bf16(dev, xb, T * cols)
    dense.cmat_mul_bf16(dev, m, xh, y, T)
    got = hip.hip_floats(y, T * rows).reshape(T, rows)[sample]
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err <= 2e-2, err
    for b in (xh, xb, y):
        hip.hip_free(b)
    act.free(); m.free()


def _full_size_experts(rng, ne, nuniq, d, ff):
    """NE experts of the full shape made of NUNIQ different ones (expert e = unique e % NUNIQ)."""
    g1 = synth.weights(synth.IQ2_XXS, nuniq * ff, d, rng)
    u1 = synth.weights(synth.IQ2_XXS, nuniq * ff, d, rng)
    d1 = synth.weights(synth.Q2_K, nuniq * d, ff, rng)
    rep = ne // nuniq
    return tuple(np.tile(a.reshape(nuniq, -1), (rep, 1)).reshape(-1) for a in (g1, u1, d1))


@pytest.mark.parametrize("clamp", [0.0, 7.0])
def test_moe_decode_step_of_config_4_with_256_experts(dev, clamp):
    """Config 4 as it is stated: 256 resident experts of the full 4096 x 2048 shape, top-6 of 256
    router logits, the shared expert in Q8_0.  The step in 12 launches, in 5, and in 6 with the
    routing left on the device (the slot table of all 256 indexed by d4_route's result) has the
    oracle's bits, with the clamp off and on."""
    from illatio_amd import ds4f, hip
    rng = synth.make_rng(4004)
    ne, d, ff, nu = 256, 4096, 2048, 6
    gate, up, down = _full_size_experts(rng, ne, 16, d, ff)
    sg = synth.weights(synth.Q8_0, ff, d, rng); su = synth.weights(synth.Q8_0, ff, d, rng)
    sd = synth.weights(synth.Q8_0, d, ff, rng)
    pool = ds4f.ExpertPool(dev, ne, d, ff, gate, up, down)
    sh = ds4f.SharedExpert(dev, d, ff, sg, su, sd)
    seen = set()
    for trial in range(3):
        norm = synth.activations(d, rng)
        logits = synth.activations(ne, rng)
        if trial == 2:
            logits[[255, 0, 128]] = 9.0                         # the table's ends, tied: the earlier index first
        want, wsel, ww = orc.moe_token(gate, up, down, sg, su, sd, d, ff, ne, nu, 1.5, clamp, logits, norm, nthreads=8)
        seen.update(wsel.tolist())
        lb, nb = hip.hip_upload_new(dev, logits), hip.hip_upload_new(dev, norm)
        sel, w = ds4f.route(dev, lb, 1, ne, nu, 1.5)
        hsel, hw = hip.hip_download(sel, np.uint32, nu), hip.hip_floats(w, nu)
        assert hsel.tolist() == wsel.tolist() and np.array_equal(bits(hw), bits(ww))
        sout = ds4f.ffn_shared(dev, sh, nb, clamp)
        moe = ds4f.ffn_tail(dev, pool, hsel, hw, nb, sout, clamp)
        fused = ds4f.ffn_step_fused(dev, pool, sh, hsel, hw, nb, clamp)
        ondev = ds4f.ffn_step_device(dev, pool, sh, lb, nb, ne, nu, 1.5, clamp)
        call = hip.hip_alloc(dev, 4 * d)                        # one call into the library: the routing over all 256 experts
        ds4f.ffn_step_call(dev, pool, sh, lb, nb, call, ne, nu, 1.5, clamp)      # carried along by the shared expert's gate/up launch
        for name, b in (("12 launches", moe), ("5 launches", fused), ("routing on the device", ondev), ("one call", call)):
            got = hip.hip_floats(b, d)
            assert np.array_equal(bits(got), bits(want)), (name, trial, np.abs(got - want).max())
        for b in (lb, nb, sel, w, sout, moe, fused, ondev, call):
            hip.hip_free(b)
    assert {0, 128, 255} <= seen and len(seen) > 12
    pool.free(); sh.free()


@pytest.mark.parametrize("clamp", [0.0, 7.0])
def test_moe_chunk_of_config_5_sampled_tokens(dev, clamp):
    """256 experts of the full 4096 x 2048 shape (16 different ones, each in 16 slots), 4096 tokens,
    top-6 with Zipf-skewed logits, the clamp off and on: the exact chunk gives every sampled token
    the bits of its own decode step, routing included.  The bf16 chunk: routing and counts equal,
    and each of the three grouped products within 2e-2 of the CPU product of the same input rows,
    on the (token, slot) rows of the sampled tokens."""
    from illatio_amd import ds4f, hip
    rng = synth.make_rng(555)
    ne, d, ff, nu, n = 256, 4096, 2048, 6, 4096
    gate, up, down = _full_size_experts(rng, ne, 16, d, ff)
    norms = synth.activations((n, d), rng)
    logits = synth.zipf_router_logits(n, ne, rng)
    shared = synth.activations((n, d), rng)
    pool = ds4f.ExpertPool(dev, ne, d, ff, gate, up, down)
    lb, nb, sb = (hip.hip_upload_new(dev, a) for a in (logits, norms, shared))
    keep = {}
    moe = ds4f.ffn_routed_chunk(dev, pool, lb, nb, sb, n, ne, nu, 1.5, clamp, keep=keep)
    got = hip.hip_floats(moe, n * d).reshape(n, d)
    assert int(keep["counts"].sum()) == n * nu
    sample = [0, 1, 63, 64, 2047, 2048, 4095]
    want, clamped = {}, 0
    for t in sample:
        sel, w = orc.route(logits[t], nu, 1.5)
        assert keep["sel"].reshape(n, nu)[t].tolist() == sel.tolist()
        assert np.array_equal(bits(keep["w"].reshape(n, nu)[t]), bits(w))
        routed, _ = orc.moe_routed(gate, up, down, d, ff, sel, w, clamp, norms[t], nthreads=8)
        if clamp:
            clamped += int(not np.array_equal(routed, orc.moe_routed(gate, up, down, d, ff, sel, w, 0.0, norms[t], nthreads=8)[0]))
        want[t] = routed + shared[t]
        assert np.array_equal(bits(got[t]), bits(want[t])), (t, np.abs(got[t] - want[t]).max())
    assert clamped == (len(sample) if clamp else 0)             # the clamp bites on every sampled token
    hip.hip_free(moe)
    exact_counts = keep["counts"]
    # bf16: the three products kept apart
    keep = {}
    moe = ds4f.ffn_routed_chunk_bf16(dev, pool, lb, nb, sb, n, ne, nu, 1.5, clamp, keep=keep)
    unfused = hip.hip_floats(moe, n * d).reshape(n, d)
    hip.hip_free(moe)
    assert np.array_equal(keep["counts"], exact_counts)
    ends = np.cumsum(keep["counts"].astype(np.int64))
    grb, drb = synth.row_bytes(synth.IQ2_XXS, d), synth.row_bytes(synth.Q2_K, ff)
    gate_e, up_e, down_e = gate.reshape(ne, ff * grb), up.reshape(ne, ff * grb), down.reshape(ne, d * drb)
    rows = np.concatenate([np.flatnonzero(keep["rmap"] == t) for t in sample])
    assert rows.size == len(sample) * nu
    cpu = {"gate": [], "up": [], "down": []}
    for r in rows:
        e = int(np.searchsorted(ends, r, side="right"))         # the group row r lies in
        assert keep["bases"][e] <= r < keep["bases"][e] + keep["counts"][e]
        xrow = norms[keep["rmap"][r]]
        cpu["gate"].append(orc.matmul(synth.IQ2_XXS, gate_e[e], ff, d, xrow, nthreads=8))
        cpu["up"].append(orc.matmul(synth.IQ2_XXS, up_e[e], ff, d, xrow, nthreads=8))
        cpu["down"].append(orc.matmul(synth.Q2_K, down_e[e], d, ff, keep["mid"][r], nthreads=8))
    for k in ("gate", "up", "down"):
        c = np.stack(cpu[k])
        err = np.abs(keep[k][rows] - c).max() / np.abs(c).max()
        assert err <= 2e-2, (k, err)                            # the tolerance the bf16 path is held to
    # gate, up and the gated activation in one launch (what the benchmark times): the same numbers
    moe = ds4f.ffn_routed_chunk_bf16(dev, pool, lb, nb, sb, n, ne, nu, 1.5, clamp)
    fused = hip.hip_floats(moe, n * d).reshape(n, d)
    assert np.array_equal(bits(fused), bits(unfused))
    for b in (lb, nb, sb, moe):
        hip.hip_free(b)
    pool.free()
