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


def test_moe_chunk_of_config_5_sampled_tokens(dev):
    """256 experts of the full 4096 x 2048 shape (16 different ones, each in 16 slots), 4096 tokens,
    top-6 with Zipf-skewed logits: the exact chunk gives every sampled token the bits of its own
    decode step, routing included; the bf16 chunk stays within 2e-2."""
    from illatio_amd import ds4f, hip
    rng = synth.make_rng(555)
    ne, nuniq, d, ff, nu, n = 256, 16, 4096, 2048, 6, 4096
    g1 = synth.weights(synth.IQ2_XXS, nuniq * ff, d, rng)
    u1 = synth.weights(synth.IQ2_XXS, nuniq * ff, d, rng)
    d1 = synth.weights(synth.Q2_K, nuniq * d, ff, rng)
    rep = ne // nuniq
    gate, up, down = (np.tile(a.reshape(nuniq, -1), (rep, 1)).reshape(-1) for a in (g1, u1, d1))
    norms = synth.activations((n, d), rng)
    logits = synth.zipf_router_logits(n, ne, rng)
    shared = synth.activations((n, d), rng)
    pool = ds4f.ExpertPool(dev, ne, d, ff, gate, up, down)
    lb, nb, sb = (hip.hip_upload_new(dev, a) for a in (logits, norms, shared))
    keep = {}
    moe = ds4f.ffn_routed_chunk(dev, pool, lb, nb, sb, n, ne, nu, 1.5, 0.0, keep=keep)
    got = hip.hip_floats(moe, n * d).reshape(n, d)
    assert int(keep["counts"].sum()) == n * nu
    sample = [0, 1, 63, 64, 2047, 2048, 4095]
    want = {}
    for t in sample:
        sel, w = orc.route(logits[t], nu, 1.5)
        assert keep["sel"].reshape(n, nu)[t].tolist() == sel.tolist()
        assert np.array_equal(bits(keep["w"].reshape(n, nu)[t]), bits(w))
        routed, _ = orc.moe_routed(gate, up, down, d, ff, sel, w, 0.0, norms[t])
        want[t] = routed + shared[t]
        assert np.array_equal(bits(got[t]), bits(want[t])), (t, np.abs(got[t] - want[t]).max())
    hip.hip_free(moe)
    moe = ds4f.ffn_routed_chunk_bf16(dev, pool, lb, nb, sb, n, ne, nu, 1.5, 0.0)
    got = hip.hip_floats(moe, n * d).reshape(n, d)
    for t in sample:
        routed = want[t] - shared[t]
        assert np.abs(got[t] - want[t]).max() <= 2e-2 * max(np.abs(routed).max(), 1e-30) * 4, t
    for b in (lb, nb, sb, moe):
        hip.hip_free(b)
    pool.free()
