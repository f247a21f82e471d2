"""A chain of dependent decode products in one launch (ilt_chain_*): a dense decoder layer's products as
cuda-forward-n strings them (cuda-dense.lisp:380-432: norm -> Q/K/V, wo with acc, norm -> gate/up with
swiglu!, down with acc), every vector handed from stage to stage on the device, against the CPU oracle's
rmsnorm!, quantizers, row dots and swiglu! composed the same way: bit for bit."""
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


def make_layers(dev, rng, nl, d, qd, kvd, ffn, dscale):
    from illatio_amd import dense, hip
    specs = [("wq", synth.Q4_K, qd, d), ("wk", synth.Q4_K, kvd, d), ("wv", synth.Q6_K, kvd, d), ("wo", synth.Q4_K, d, qd),
             ("gate", synth.Q4_K, ffn, d), ("up", synth.Q4_K, ffn, d), ("down", synth.Q6_K, d, ffn)]
    layers = []
    for li in range(nl):
        host = {n: synth.weights(t, r, c, rng, dscale=dscale[t]) for n, t, r, c in specs}
        L = {"host": host, "dev": {n: dense.upload_gmat(dev, n, t, r, c, host[n]) for n, t, r, c in specs}}
        for n in ("attn_norm", "ffn_norm"):
            L[n] = (synth.activations(d, rng) * 0.2 + 1.0).astype(np.float32)
            L[n + "_dev"] = hip.hip_upload_new(dev, L[n])
        L["bq"] = synth.activations(qd, rng)
        L["bq_dev"] = hip.hip_upload_new(dev, L["bq"])
        layers.append(L)
    return specs, layers


def cpu_chain(layers, x, d, qd, kvd, ffn, eps, nthreads=8):
    """The chain on the CPU: what each stage's output must be."""
    outs = []
    for L in layers:
        h = L["host"]
        xn = orc.rmsnorm(x, L["attn_norm"], eps)
        q = orc.matmul(synth.Q4_K, h["wq"], qd, d, xn, nthreads=nthreads) + L["bq"]
        k = orc.matmul(synth.Q4_K, h["wk"], kvd, d, xn, nthreads=nthreads)
        v = orc.matmul(synth.Q6_K, h["wv"], kvd, d, xn, nthreads=nthreads)
        x1 = x + orc.matmul(synth.Q4_K, h["wo"], d, qd, q, nthreads=nthreads)          # attention stood in for by q itself
        hn = orc.rmsnorm(x1, L["ffn_norm"], eps)
        mid = orc.swiglu(orc.matmul(synth.Q4_K, h["gate"], ffn, d, hn, nthreads=nthreads),
                         orc.matmul(synth.Q4_K, h["up"], ffn, d, hn, nthreads=nthreads))
        x2 = x1 + orc.matmul(synth.Q6_K, h["down"], d, ffn, mid, nthreads=nthreads)
        outs.append({"q": q, "k": k, "v": v, "x1": x1, "mid": mid, "x2": x2})
        x = x2
    return outs


def build_chain(dev, layers, xb, d, qd, kvd, ffn, eps, keep_all):
    from illatio_amd import dense, hip
    stages, bufs = [], []
    x_src, r_src = xb, xb
    for L in layers:
        D = L["dev"]
        y = {n: hip.hip_alloc(dev, 4 * r) for n, r in (("q", qd), ("k", kvd), ("v", kvd), ("x1", d), ("mid", ffn), ("x2", d))}
        bufs.append(y)
        s0 = len(stages)
        stages.append(dense.chain_stage([(D["wq"], y["q"], L["bq_dev"]), (D["wk"], y["k"], None), (D["wv"], y["v"], None)], x_src,
                                        norm=(L["attn_norm_dev"], eps)))
        stages.append(dense.chain_stage([(D["wo"], y["x1"] if keep_all else None, None)], (s0, 0), resid=r_src))
        stages.append(dense.chain_stage([(D["gate"], y["mid"] if keep_all else None, None), (D["up"], None, None)], (s0 + 1, 0), glu=True,
                                        norm=(L["ffn_norm_dev"], eps)))
        stages.append(dense.chain_stage([(D["down"], y["x2"], None)], (s0 + 2, 0), resid=(s0 + 1, 0)))
        x_src = r_src = (s0 + 3, 0)
    return dense.Chain(dev, stages), bufs


@pytest.mark.parametrize("nl,d,qd,kvd,ffn", [(3, 512, 768, 256, 1280),        # a few rows a CU
                                             (2, 256, 256, 100, 512),          # K and V of fewer rows than CUs: workgroups with no rows of them, ragged shares
                                             (2, 2560, 4096, 1024, 9728)])     # config 2's layer: 38 rows of gate and up a CU, 38 blocks a down row
def test_chain_of_layers_bit_exact(dev, nl, d, qd, kvd, ffn):
    from illatio_amd import hip
    rng = synth.make_rng(nl * 1000 + d)
    # scales that keep the stream's magnitude within a few orders over the layers
    specs, layers = make_layers(dev, rng, nl, d, qd, kvd, ffn, {synth.Q4_K: 0.0005, synth.Q6_K: 0.0003})
    eps = 1e-6
    x = synth.activations(d, rng)
    xb = hip.hip_upload_new(dev, x)
    chain, bufs = build_chain(dev, layers, xb, d, qd, kvd, ffn, eps, keep_all=True)
    want = cpu_chain(layers, x, d, qd, kvd, ffn, eps)
    for run in range(3):                     # the tags move on from run to run; the words of the run before are stale
        chain.run()
        assert chain.status() == 0
        for li, (y, w) in enumerate(zip(bufs, want)):
            for n in ("q", "k", "v", "x1", "mid", "x2"):
                got = hip.hip_floats(y[n], w[n].size)
                assert np.array_equal(bits(got), bits(w[n])), (run, li, n, np.abs(got - w[n]).max())
                if run < 2:
                    hip.hip_zero(y[n])
    # another input through the same chain
    x = synth.activations(d, rng) * np.float32(3.0)
    hip.hip_upload_vector(xb, x)
    want = cpu_chain(layers, x, d, qd, kvd, ffn, eps)
    chain.run()
    assert chain.status() == 0
    got = hip.hip_floats(bufs[-1]["x2"], d)
    assert np.array_equal(bits(got), bits(want[-1]["x2"]))
    chain.free()


def test_chain_rejects_what_it_cannot_hold(dev):
    from illatio_amd import dense, hip
    rng = synth.make_rng(5)
    w = synth.weights(synth.Q4_K, 64, 256, rng)
    m = dense.upload_gmat(dev, "w", synth.Q4_K, 64, 256, w)
    big = dense.CMat("big", synth.Q4_K, 1 << 20, 4096, m.qs)            # 2.4 GB "matrix": 9.4 MB a CU
    xb, y = hip.hip_upload_new(dev, synth.activations(256, rng)), hip.hip_alloc(dev, 4 * 64)
    with pytest.raises(hip.HipError):
        dense.Chain(dev, [dense.chain_stage([(big, None, None)], xb)])
    with pytest.raises(hip.HipError):                                   # an input of the wrong length
        dense.Chain(dev, [dense.chain_stage([(m, y, None)], xb), dense.chain_stage([(m, y, None)], (0, 0))])
    with pytest.raises(hip.HipError):                                   # a stage reading a later one
        dense.Chain(dev, [dense.chain_stage([(m, y, None)], (0, 0))])
    for b in (xb, y):
        hip.hip_free(b)
    m.free()
