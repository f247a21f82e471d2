"""The dense decoder on the device against the CPU oracle's forward-1 (model.lisp:396-462): random-init models of
the benchmark's config 2 family (Q4_K / Q6_K, head norms, neox RoPE, grouped-query attention), a prompt through
the prefill products in chunks, then a greedy decode.  Every product is bit-exact and the kernels between them add
in the CPU's order, so each step's logits are compared bit for bit; the greedy token is then the CPU path's without
any near-tie allowance (the reference's own GPU tests allow one, cuda-consistency-test.lisp:19-22, because its
CUDA kernels add in another order)."""
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


def run_greedy(dev, host, nprompt, ndecode, chunk, nctx, seed, check_cache=False, one_call=True, say=None):
    from illatio_amd import hip, model
    c = host["config"]
    rng = synth.make_rng(seed)
    prompt = rng.integers(0, c["vocab"], nprompt).tolist()
    cpu = orc.DenseModel(host, nctx)
    for i, t in enumerate(prompt[:-1]):
        cpu.forward(t, logits=False, nthreads=16)
        if say and i % 64 == 63:
            say(f"oracle: prompt position {i + 1} of {nprompt}")
    want, _ = cpu.forward(prompt[-1], nthreads=16)
    gpu = model.DenseModel(dev, host, nctx, chunk=chunk)
    gpu.one_call = gpu.one_call and one_call                  # a token by ilt_dense_decode, or launch by launch from Python
    gpu.eval_tokens(prompt)                                   # the prompt through the prefill products, chunk by chunk
    got = hip.hip_floats(gpu.logits, c["vocab"])
    assert np.array_equal(bits(got), bits(want)), ("prompt", np.abs(got - want).max())
    if check_cache:                                           # batched prefill leaves the caches token-at-a-time decoding leaves
        kvd = c["nkv"] * c["hd"]
        for li in (0, c["nl"] - 1):
            for name, ref in (("kc", cpu.kc), ("vc", cpu.vc)):
                dv = hip.hip_floats(gpu.layers[li][name], nprompt * kvd).reshape(nprompt, kvd)
                assert np.array_equal(bits(dv), bits(ref[li, :nprompt])), (li, name)
    same, margins = 0, []
    for step in range(ndecode):
        tok = int(np.argmax(want))
        assert gpu.argmax() == tok, step
        top2 = np.partition(want, -2)[-2:]
        margins.append(float(top2[1] - top2[0]))
        want, _ = cpu.forward(tok, nthreads=16)
        gpu.forward_n([tok])                                  # one token: the decode products
        got = hip.hip_floats(gpu.logits, c["vocab"])
        assert np.array_equal(bits(got), bits(want)), (step, np.abs(got - want).max())
        same += 1
        if say and step % 32 == 31:
            say(f"greedy token {step + 1} of {ndecode}: logits bit for bit, smallest top-1 margin so far {min(margins):.4f}")
    gpu.free()
    return same, margins


def test_small_decoder_prefill_chunks_and_decode(dev):
    from illatio_amd import model
    host = model.synth_model(3, d=512, ffn=1024, nh=8, nkv=2, hd=64, nl=3, vocab=1000)
    same, _ = run_greedy(dev, host, nprompt=40, ndecode=24, chunk=16, nctx=80, seed=1, check_cache=True)
    assert same == 24
    same, _ = run_greedy(dev, host, nprompt=40, ndecode=24, chunk=16, nctx=80, seed=1, one_call=False)
    assert same == 24
    # a prompt of one token, and a chunk larger than the prompt
    run_greedy(dev, host, nprompt=1, ndecode=3, chunk=16, nctx=8, seed=2)
    run_greedy(dev, host, nprompt=9, ndecode=2, chunk=64, nctx=16, seed=3)


@pytest.mark.parametrize("norms,nh,nkv,hd", [(True, 8, 2, 64), (False, 8, 2, 64), (True, 3, 1, 64), (True, 4, 2, 32)])
def test_attn_step_is_qk_rope_then_attn_rows(dev, norms, nh, nkv, hd):
    """One token's attention as one launch (heads of 64) or two (heads of 32) (ilt_attn_step) against the three it
    stands for, at positions in the first and in later blocks of 256 scores and on a block's edges: the output and the
    caches' rows bit for bit, q and k untouched."""
    import ctypes as C
    from illatio_amd import hip
    nctx, eps = 600, 1e-6                             # (3 heads: 12 workgroups, not a multiple of the eight dies)
    rng = synth.make_rng(11)
    f = lambda *sh: (rng.standard_normal(sh) * 1.5).astype(np.float32)
    up = lambda a: (lambda b: (hip.hip_upload_vector(b, a), b)[1])(hip.hip_alloc(dev, a.nbytes))
    P = lambda b: C.c_uint64(b.ptr if b is not None else 0)
    S = C.c_uint64(0)
    table = np.zeros((nctx, hd), np.float32)
    assert hip.lib().ilt_rope_table(C.c_int(hd), C.c_int(0), C.c_int(nctx), C.c_float(1e6), table.ctypes.data_as(C.c_void_p)) == 0
    rope, qn, kn = up(table), (up(f(hd)) if norms else None), (up(f(hd)) if norms else None)
    kc0, vc0 = f(nctx, nkv * hd), f(nctx, nkv * hd)
    scratch = hip.hip_alloc(dev, 4 * nh * nctx)
    for pos in (0, 1, 255, 256, 257, 511, 599):
        q, k, v = f(nh * hd), f(nkv * hd), f(nkv * hd)
        res = []
        for fused in (False, True):
            dq, dk, dv, kc, vc, out = up(q), up(k), up(v), up(kc0), up(vc0), hip.hip_alloc(dev, 4 * nh * hd)
            ints = (C.c_int(nh), C.c_int(nkv), C.c_int(hd), C.c_int(hd), C.c_int(pos), C.c_float(eps), C.c_int(1))
            if fused:
                hip.call("ilt_attn_step", S, P(dq), P(dk), P(dv), P(qn), P(kn), P(rope), P(kc), P(vc), P(out), *ints, P(scratch), C.c_int(nctx))
                assert np.array_equal(bits(hip.hip_floats(dq, nh * hd)), bits(q)) and np.array_equal(bits(hip.hip_floats(dk, nkv * hd)), bits(k))
            else:
                hip.call("ilt_qk_rope", S, P(dq), P(dk), P(dv), P(qn), P(kn), P(rope), P(kc), P(vc), *ints, C.c_int(1))
                hip.call("ilt_attn_rows", S, P(dq), P(kc), P(vc), P(out), C.c_int(nh), C.c_int(nkv), C.c_int(hd), C.c_int(pos), C.c_int(1), P(None))
            res.append([hip.hip_floats(b, n) for b, n in ((out, nh * hd), (kc, nctx * nkv * hd), (vc, nctx * nkv * hd))])
            for b in (dq, dk, dv, kc, vc, out):
                hip.hip_free(b)
        for a, b, what in zip(res[0], res[1], ("out", "kc", "vc")):
            assert np.array_equal(bits(a), bits(b)), (pos, what)
        assert not np.array_equal(res[0][1], kc0.ravel())         # the key's row was written
    # a position the caches have no row for is refused
    dq, dk, dv, kc, vc, out = up(f(nh * hd)), up(f(nkv * hd)), up(f(nkv * hd)), up(kc0), up(vc0), hip.hip_alloc(dev, 4 * nh * hd)
    with pytest.raises(hip.HipError):
        hip.call("ilt_attn_step", S, P(dq), P(dk), P(dv), P(qn), P(kn), P(rope), P(kc), P(vc), P(out), C.c_int(nh), C.c_int(nkv), C.c_int(hd),
                 C.c_int(hd), C.c_int(nctx), C.c_float(eps), C.c_int(1), P(scratch), C.c_int(nctx))
    for b in (dq, dk, dv, kc, vc, out):
        hip.hip_free(b)
    for b in (rope, qn, kn, scratch):
        hip.hip_free(b)


def test_the_reference_attention_names_launch(dev):
    """attn_decode + attn_merge and attn_prefill / attn_prefill2 by the reference's names and argument lists
    (cuda-dense.lisp:341-364): the heads they leave are attn_rows' -- the CPU's float order -- and attn_merge's
    quantized copy is quant_q8's of them."""
    from illatio_amd import hip
    nh, nkv, hd, nctx = 8, 2, 64, 300
    rng = synth.make_rng(21)
    f = lambda *sh: (rng.standard_normal(sh) * 1.5).astype(np.float32)
    up = lambda a: hip.hip_upload_new(dev, a)
    kc, vc = up(f(nctx, nkv * hd)), up(f(nctx, nkv * hd))
    scale = float(1.0 / np.sqrt(hd))
    # one token at position 200
    q = up(f(nh * hd))
    part, att, want = (hip.hip_alloc(dev, 4 * nh * (hd + 2) * 8) for _ in range(3))
    xq, xs, xsum = hip.hip_alloc(dev, nh * hd), hip.hip_alloc(dev, 4 * nh * hd // 32), hip.hip_alloc(dev, 4 * nh * hd // 32)
    hip.launch(dev, "attn_decode", (nkv, 4), 128, [q, kc, vc, part, nh, nkv, hd, 200, 64, 4, scale], shared=4096)
    hip.launch(dev, "attn_merge", (nh, 1), 64, [part, att, xq, xs, xsum, nh, hd, 200, 64, 4])
    hip.launch(dev, "attn_rows", (nh, 1), 256, [q, kc, vc, want, nh, nkv, hd, 200, None])
    w = hip.hip_floats(want, nh * hd)
    assert np.array_equal(bits(hip.hip_floats(att, nh * hd)), bits(w))
    wq, ws_, wsum = hip.hip_alloc(dev, nh * hd), hip.hip_alloc(dev, 4 * nh * hd // 32), hip.hip_alloc(dev, 4 * nh * hd // 32)
    hip.launch(dev, "quant_q8", 1, 256, [want, wq, ws_, wsum, hip.I64(nh * hd // 32)])
    for got, ref, dt, n in ((xq, wq, np.int8, nh * hd), (xs, ws_, np.float32, nh * hd // 32), (xsum, wsum, np.int32, nh * hd // 32)):
        assert np.array_equal(hip.hip_download(got, dt, n), hip.hip_download(ref, dt, n))
    # a chunk of 37 tokens at positions 100..136, both names
    n = 37
    qn = up(f(n, nh * hd))
    for name, extra in (("attn_prefill2", []), ("attn_prefill", [4])):
        out, ref = hip.hip_alloc(dev, 4 * n * nh * hd), hip.hip_alloc(dev, 4 * n * nh * hd)
        hip.launch(dev, name, (nh, 1), 256, [qn, kc, vc, out, nh, nkv, hd, 100, n, scale] + extra, shared=8192)
        hip.launch(dev, "attn_rows", (nh, n), 256, [qn, kc, vc, ref, nh, nkv, hd, 100, None])
        assert np.array_equal(bits(hip.hip_floats(out, n * nh * hd)), bits(hip.hip_floats(ref, n * nh * hd))), name
        hip.hip_free(out); hip.hip_free(ref)
    for b in (kc, vc, q, part, att, want, xq, xs, xsum, wq, ws_, wsum, qn):
        hip.hip_free(b)


def test_attn_step_replayed_from_a_graph(dev):
    """The one-launch attention with the scores shared out keeps its flags' generation on the device: a launch captured
    into a HIP graph and replayed (new q, k, v each time, the program's own copies and waits between the replays) gives
    what the three launches it stands for give, every time."""
    import ctypes as C
    from illatio_amd import hip
    rt = C.CDLL("libamdhip64.so")
    nh, nkv, hd, nctx, pos, eps = 8, 2, 64, 400, 300, 1e-6
    rng = synth.make_rng(12)
    f = lambda *sh: (rng.standard_normal(sh) * 1.5).astype(np.float32)
    up = lambda a: (lambda b: (hip.hip_upload_vector(b, a), b)[1])(hip.hip_alloc(dev, a.nbytes))
    P = lambda b: C.c_uint64(b.ptr if b is not None else 0)
    table = np.zeros((nctx, hd), np.float32)
    assert hip.lib().ilt_rope_table(C.c_int(hd), C.c_int(0), C.c_int(nctx), C.c_float(1e6), table.ctypes.data_as(C.c_void_p)) == 0
    rope, qn, kn = up(table), up(f(hd)), up(f(hd))
    kc0, vc0 = f(nctx, nkv * hd), f(nctx, nkv * hd)
    scratch = hip.hip_alloc(dev, 4 * nh * nctx)
    q, k, v = f(nh * hd), f(nkv * hd), f(nkv * hd)
    dq, dk, dv, kc, vc, out = up(q), up(k), up(v), up(kc0), up(vc0), hip.hip_alloc(dev, 4 * nh * hd)
    ints = (C.c_int(nh), C.c_int(nkv), C.c_int(hd), C.c_int(hd), C.c_int(pos), C.c_float(eps), C.c_int(1))
    S = C.c_uint64(dev.stream)
    step = lambda: hip.call("ilt_attn_step", S, P(dq), P(dk), P(dv), P(qn), P(kn), P(rope), P(kc), P(vc), P(out), *ints, P(scratch), C.c_int(nctx))
    step()                                             # once outside the graph: the kernel's attributes are set on its first launch
    hip.hip_sync(dev)
    graph, gexec = C.c_void_p(), C.c_void_p()
    assert rt.hipStreamBeginCapture(C.c_void_p(dev.stream), C.c_int(0)) == 0
    step()
    assert rt.hipStreamEndCapture(C.c_void_p(dev.stream), C.byref(graph)) == 0
    assert rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
    for rep in range(4):
        q, k, v = f(nh * hd), f(nkv * hd), f(nkv * hd)
        for b, a in ((dq, q), (dk, k), (dv, v), (kc, kc0), (vc, vc0)):
            hip.hip_upload_vector(b, a)
        hip.hip_sync(dev)
        assert rt.hipGraphLaunch(gexec, C.c_void_p(dev.stream)) == 0
        hip.hip_sync(dev)
        got = [hip.hip_floats(b, n) for b, n in ((out, nh * hd), (kc, nctx * nkv * hd))]
        eq, ek, ev, ekc, evc, eout = up(q), up(k), up(v), up(kc0), up(vc0), hip.hip_alloc(dev, 4 * nh * hd)
        hip.call("ilt_qk_rope", S, P(eq), P(ek), P(ev), P(qn), P(kn), P(rope), P(ekc), P(evc), *ints, C.c_int(1))
        hip.call("ilt_attn_rows", S, P(eq), P(ekc), P(evc), P(eout), C.c_int(nh), C.c_int(nkv), C.c_int(hd), C.c_int(pos), C.c_int(1), P(None))
        want = [hip.hip_floats(b, n) for b, n in ((eout, nh * hd), (ekc, nctx * nkv * hd))]
        for a, b, what in zip(got, want, ("out", "kc")):
            assert np.array_equal(bits(a), bits(b)), (rep, what)
        for b in (eq, ek, ev, ekc, evc, eout):
            hip.hip_free(b)
    assert rt.hipGraphExecDestroy(gexec) == 0 and rt.hipGraphDestroy(graph) == 0
    for b in (rope, qn, kn, scratch, dq, dk, dv, kc, vc, out):
        hip.hip_free(b)


def test_argmax_on_the_device(dev):
    """ilt_argmax against ARGMAX's scan (model.lisp:464-468): the first of equal maxima, -0 and +0 equal, a NaN never
    greater, a NaN in front staying the best, nothing but -inf or NaN leaving index 0; lengths that are and are not
    multiples of four."""
    import ctypes as C
    from illatio_amd import hip
    def scan(v):
        best = 0
        for i in range(len(v)):
            if v[i] > v[best]:
                best = i
        return best
    rng = synth.make_rng(99)
    out, scratch = hip.hip_alloc(dev, 4), hip.hip_alloc(dev, 2048)
    cases = []
    for n in (1, 3, 4, 1000, 4099, 151936):
        v = rng.standard_normal(n).astype(np.float32)
        cases.append(v)
        w = v.copy(); w[n // 2:] = v.max(); cases.append(w)                      # many equal maxima: the first
        w = v.copy(); w[-1] = np.inf; cases.append(w)
        w = v.copy(); w[::3] = np.nan; cases.append(w)                           # a NaN in front
        if n > 4:
            w = v.copy(); w[1::3] = np.nan; w[5] = 100.0; cases.append(w)        # NaNs elsewhere
    cases += [np.full(70, -np.inf, np.float32), np.full(9, np.nan, np.float32), np.array([-0.0, 0.0, -0.0], np.float32),
              np.array([-np.inf, -np.inf, 1.0, 1.0], np.float32), np.array([2.0, np.nan, 2.0, 3.0, np.nan, 3.0], np.float32)]
    for v in cases:
        b = hip.hip_upload_new(dev, v)
        for sc in (0, scratch.ptr):                                              # one workgroup; 128 and a second launch
            hip.call("ilt_argmax", C.c_uint64(dev.stream), C.c_uint64(b.ptr), C.c_int(len(v)), C.c_uint64(out.ptr), C.c_uint64(sc))
            got = int(hip.hip_download(out, np.int32, 1)[0])
            with np.errstate(invalid="ignore"):
                assert got == scan(v), (len(v), got, scan(v), sc != 0)
        hip.hip_free(b)
    hip.hip_free(out)
    hip.hip_free(scratch)


def test_greedy_decode_on_the_device(dev):
    """decode_greedy: the tokens picked on the device and fed on from device memory are the tokens the oracle's greedy
    decode picks, and the logits after the last of them have the oracle's bits."""
    from illatio_amd import hip, model
    host = model.synth_model(12, d=512, ffn=1024, nh=8, nkv=2, hd=64, nl=2, vocab=777)
    rng = synth.make_rng(12)
    prompt = rng.integers(0, 777, 19).tolist()
    cpu = orc.DenseModel(host, 64)
    for t in prompt[:-1]:
        cpu.forward(t, logits=False, nthreads=8)
    want, _ = cpu.forward(prompt[-1], nthreads=8)
    gpu = model.DenseModel(dev, host, 64, chunk=8)
    gpu.eval_tokens(prompt)
    ids = gpu.decode_greedy(30)
    expect = []
    for _ in range(30):
        tok = int(np.argmax(want))
        expect.append(tok)
        want, _ = cpu.forward(tok, nthreads=8)
    assert ids == expect
    assert np.array_equal(bits(hip.hip_floats(gpu.logits, 777)), bits(want))
    gpu.free()


def test_reused_context_is_a_fresh_one(dev):
    """A context used for one sequence, reset and used for another gives the second the logits a fresh context gives
    (the reference's consistency-test.lisp:52-61): nothing of the first sequence's caches or buffers shows."""
    from illatio_amd import hip, model
    host = model.synth_model(10, d=512, ffn=1024, nh=8, nkv=2, hd=64, nl=2, vocab=600)
    rng = synth.make_rng(10)
    first, second = rng.integers(0, 600, 50).tolist(), rng.integers(0, 600, 23).tolist()
    gpu = model.DenseModel(dev, host, 64, chunk=16)
    gpu.eval_tokens(first)
    for _ in range(5):
        gpu.forward_n([gpu.argmax()])
    gpu.reset()
    gpu.eval_tokens(second)
    reused = hip.hip_floats(gpu.logits, 600).copy()
    gpu.free()
    fresh = model.DenseModel(dev, host, 64, chunk=16)
    fresh.eval_tokens(second)
    assert np.array_equal(bits(reused), bits(hip.hip_floats(fresh.logits, 600)))
    cpu = orc.DenseModel(host, 64)
    for t in second[:-1]:
        cpu.forward(t, logits=False, nthreads=8)
    want, _ = cpu.forward(second[-1], nthreads=8)
    assert np.array_equal(bits(reused), bits(want))
    fresh.free()


def test_llama_style_decoder(dev):
    """No head norms, RoPE on adjacent pairs (2i, 2i + 1), heads of 96 (six partial sums of sixteen a score), one KV
    head for all query heads; then heads of 256, the widest the attention takes."""
    from illatio_amd import model
    host = model.synth_model(8, d=512, ffn=768, nh=8, nkv=1, hd=96, nl=2, vocab=400)
    host["config"]["neox"] = False
    for L in host["layers"]:
        L["q_norm"] = L["k_norm"] = None
    for one_call in (True, False):
        same, _ = run_greedy(dev, host, nprompt=21, ndecode=8, chunk=8, nctx=40, seed=8, check_cache=True, one_call=one_call)
        assert same == 8
    host = model.synth_model(9, d=512, ffn=768, nh=2, nkv=2, hd=256, nl=1, vocab=400)
    same, _ = run_greedy(dev, host, nprompt=300, ndecode=4, chunk=64, nctx=320, seed=9)
    assert same == 4


def test_qwen2_style_q8_decoder(dev):
    """The config 1 family: every matrix Q8_0 (activations in Q8_0 blocks with the scale through fp16), biases on Q, K
    and V, no head norms -- a small model with the prompt in chunks and both ways of queueing a token, then config 1's
    own widths (896 / 4864, 14 query heads on 2 KV heads of 64, the full vocabulary), two layers."""
    from illatio_amd import model
    host = model.synth_model_q8(31, d=512, ffn=1024, nh=8, nkv=2, hd=64, nl=2, vocab=600)
    assert host["layers"][0]["bq"] is not None and host["layers"][0]["q_norm"] is None
    same, _ = run_greedy(dev, host, nprompt=20, ndecode=12, chunk=8, nctx=40, seed=31, check_cache=True)
    assert same == 12
    same, _ = run_greedy(dev, host, nprompt=20, ndecode=6, chunk=8, nctx=40, seed=32, one_call=False)
    assert same == 6
    host = model.synth_model_q8(33, nl=2)
    same, margins = run_greedy(dev, host, nprompt=40, ndecode=24, chunk=32, nctx=70, seed=33)
    assert same == 24 and min(margins) > 0


def test_small_decoder_long_contexts(dev):
    """Contexts past one workgroup's 256 positions of scores: the two-launch attention with 16 tokens, 4 tokens and one
    token a workgroup as the context grows towards 2048 positions, and past that the value slice in tiles."""
    from illatio_amd import model
    host = model.synth_model(6, d=256, ffn=512, nh=4, nkv=2, hd=64, nl=2, vocab=500)
    same, _ = run_greedy(dev, host, nprompt=2030, ndecode=6, chunk=512, nctx=2040, seed=6)
    assert same == 6
    same, _ = run_greedy(dev, host, nprompt=2060, ndecode=4, chunk=512, nctx=2100, seed=7)
    assert same == 4
    # past 2048 positions the value slice goes through LDS in tiles of 1024 positions: four tokens a workgroup up to
    # 4096 positions, one beyond; the decode steps cross a tile's edge (4096 -> 4097)
    same, _ = run_greedy(dev, host, nprompt=4094, ndecode=6, chunk=512, nctx=4110, seed=13)
    assert same == 6
    same, _ = run_greedy(dev, host, nprompt=4400, ndecode=3, chunk=512, nctx=4410, seed=14, one_call=False)
    assert same == 3
    # one token's values past 2,048 positions come in tiles of 480 positions while the chains run: the decode steps cross
    # a tile's edge (2,400 -> 2,401), with an even and with an odd number of tiles
    same, _ = run_greedy(dev, host, nprompt=2397, ndecode=6, chunk=2048, nctx=2410, seed=15)      # (a chunk of 2,048 tokens, then 349)
    assert same == 6
    same, _ = run_greedy(dev, host, nprompt=2878, ndecode=5, chunk=512, nctx=2890, seed=16)
    assert same == 5
    # 1,025 to 2,048 positions: the same kernel by default (1,438 -> 1,441: a tile's edge); launch by launch from Python
    # the values' whole slice goes into LDS first (attn_rows' kernels of one token)
    same, _ = run_greedy(dev, host, nprompt=1436, ndecode=6, chunk=512, nctx=1450, seed=17)
    assert same == 6
    same, _ = run_greedy(dev, host, nprompt=1500, ndecode=3, chunk=512, nctx=1510, seed=18, one_call=False)
    assert same == 3


def test_chunk_attention_on_the_kernels_of_16_tokens(dev, monkeypatch):
    """The kernels a chunk's values went through before the 32 x 32 one, still taken by heads whose width is not a multiple
    of 32 (and, with ILT_ATTN_CHUNK=0, by any): whole in LDS up to about 1,100 positions, in tiles past that; and heads of
    48, whose score kernel reads the head's width at run time."""
    from illatio_amd import model
    host = model.synth_model(8, d=256, ffn=512, nh=16, nkv=4, hd=48, nl=2, vocab=400)      # (16 x 48 = 768 columns for wo: whole super-blocks)
    same, _ = run_greedy(dev, host, nprompt=300, ndecode=3, chunk=128, nctx=310, seed=21)
    assert same == 3
    same, _ = run_greedy(dev, host, nprompt=1300, ndecode=2, chunk=256, nctx=1310, seed=22)
    assert same == 2
    monkeypatch.setenv("ILT_ATTN_CHUNK", "0")
    host = model.synth_model(9, d=256, ffn=512, nh=4, nkv=2, hd=64, nl=2, vocab=400)
    same, _ = run_greedy(dev, host, nprompt=1300, ndecode=2, chunk=256, nctx=1310, seed=23)
    assert same == 2


@pytest.mark.parametrize("nh,nkv,hd,pos0,ntok", [(8, 2, 128, 0, 100), (8, 2, 128, 300, 77), (3, 1, 128, 37, 33), (8, 2, 64, 0, 130),
                                                 (6, 2, 64, 500, 65), (16, 4, 128, 1536, 512), (8, 8, 64, 31, 1)])
def test_chunk_attention_with_sixteen_scores_and_chains_a_thread(dev, monkeypatch, nh, nkv, hd, pos0, ntok):
    """A chunk's attention through the scores kernel of four tokens x four positions a thread, softmax and the values kernel
    of four tokens x four columns a thread (heads of 64 and 128) against attn_rows' one launch (a workgroup a head and token, the CPU's float order from end to end) and
    against the values kernel of one chain a thread: bit for bit; chunks that end inside a token tile, that start at a
    position that is no multiple of the position tile, heads that do not fill the eight dies, one token."""
    import ctypes as C
    from illatio_amd import hip
    rng = synth.make_rng(1000 + nh + hd + pos0 + ntok)
    f = lambda *sh: (rng.standard_normal(sh) * 1.5).astype(np.float32)
    nctx = pos0 + ntok
    q, kc, vc = (hip.hip_upload_new(dev, a) for a in (f(ntok, nh * hd), f(nctx, nkv * hd), f(nctx, nkv * hd)))
    smax = (nctx + 3) & ~3
    scratch = hip.hip_alloc(dev, 4 * ntok * nh * smax)
    P = lambda b: C.c_uint64(b.ptr if b is not None else 0)
    ints = (C.c_int(nh), C.c_int(nkv), C.c_int(hd), C.c_int(pos0), C.c_int(ntok))
    outs = []
    for scr, quad in ((None, None), (scratch, "1"), (scratch, "v"), (scratch, "0")):      # "v": only the values on the new kernel
        if quad is not None:
            monkeypatch.setenv("ILT_ATTN_QUAD", quad)
        out = hip.hip_upload_new(dev, np.full(ntok * nh * hd, np.nan, np.float32))
        hip.call("ilt_attn_rows", C.c_uint64(0), P(q), P(kc), P(vc), P(out), *ints, P(scr))
        outs.append(hip.hip_floats(out, ntok * nh * hd))
        hip.hip_free(out)
    assert not np.isnan(outs[0]).any()
    assert np.array_equal(bits(outs[1]), bits(outs[0])), np.abs(outs[1] - outs[0]).max()
    assert np.array_equal(bits(outs[2]), bits(outs[0])) and np.array_equal(bits(outs[3]), bits(outs[0]))
    for b in (q, kc, vc, scratch):
        hip.hip_free(b)


def test_a_chunk_as_parts_side_by_side(dev):
    """forward_parts -- a chunk's halves or quarters on streams of their own, a part's attention waiting for the earlier
    parts' keys layer by layer -- leaves forward_n's logits and caches, bit for bit: halves of 128 + 128, of 256 + 44 (the
    second half on the products for few tokens), a second chunk whose halves see the first chunk's positions, and
    quarters of 128."""
    from illatio_amd import hip, model
    host = model.synth_model(12, d=512, ffn=1024, nh=8, nkv=2, hd=64, nl=3, vocab=700)
    c = host["config"]
    rng = synth.make_rng(77)
    kvd = c["nkv"] * c["hd"]
    for nprompt, chunk, k in ((256, 256, 2), (300, 300, 2), (600, 300, 2), (512, 512, 4), (1000, 500, 4), (1000, 1000, 2)):
        prompt = rng.integers(0, c["vocab"], nprompt).tolist()
        res = []
        for halves in (True, False):
            m = model.DenseModel(dev, host, nctx=nprompt + 8, chunk=chunk)
            for i in range(0, nprompt, chunk):
                part = prompt[i:i + chunk]
                if halves:
                    m.forward_parts(part, logits=i + chunk >= nprompt, k=k)
                else:
                    m.forward_n(part, logits=i + chunk >= nprompt)
            hip.hip_sync(dev)
            assert m.pos == nprompt
            res.append([hip.hip_floats(m.logits, c["vocab"])] + [hip.hip_floats(m.layers[li][nm], nprompt * kvd) for li in (0, 2) for nm in ("kc", "vc")])
            m.free()
        for a, b in zip(*res):
            assert np.array_equal(bits(a), bits(b)), (nprompt, chunk)


def test_bf16_chunk_as_halves_stays_within_the_bf16_roundings(dev):
    """The bf16 prefill through forward_parts: the halves' products are other launches (other token counts, so the
    split over the columns may fall otherwise), not other numbers -- the first layer's caches within a few bf16 roundings of the whole
    chunk's, the logits within 2e-2 of their spread."""
    from illatio_amd import hip, model
    host = model.synth_model(13, d=512, ffn=1024, nh=8, nkv=2, hd=64, nl=3, vocab=700)
    c = host["config"]
    rng = synth.make_rng(78)
    nprompt, kvd = 1024, c["nkv"] * c["hd"]
    prompt = rng.integers(0, c["vocab"], nprompt).tolist()
    res = []
    for parts in (True, False):
        m = model.DenseModel(dev, host, nctx=nprompt + 8, chunk=nprompt, prefill="bf16")
        if parts:
            m.forward_parts(prompt, k=2)
        else:
            m.forward_n(prompt)
        hip.hip_sync(dev)
        res.append((hip.hip_floats(m.logits, c["vocab"]), hip.hip_floats(m.layers[0]["kc"], nprompt * kvd), hip.hip_floats(m.layers[0]["vc"], nprompt * kvd)))
        m.free()
    (la, ka, va), (lb, kb, vb) = res
    assert np.abs(ka - kb).max() <= 2e-2 * np.abs(kb).max() and np.abs(va - vb).max() <= 2e-2 * np.abs(vb).max()
    assert np.abs(la - lb).max() <= 2e-2 * lb.std(), (np.abs(la - lb).max(), lb.std())


def test_chunk_attention_on_seeded_random_shapes(dev):
    """The same comparison on a dozen seeded shapes: heads of 64 and 128, 1 to 12 query heads on 1 to 4 KV heads, chunks
    of 2 to 300 tokens starting anywhere up to 3,000 positions, and one chunk that ends at position 8,192."""
    import ctypes as C
    from illatio_amd import hip
    rng = synth.make_rng(4242)
    shapes = []
    for _ in range(11):
        nkv = int(rng.integers(1, 5)); nh = nkv * int(rng.integers(1, 4)); hd = int(rng.choice([64, 128]))
        shapes.append((nh, nkv, hd, int(rng.integers(0, 3000)), int(rng.integers(2, 301))))
    shapes.append((2, 1, 128, 8192 - 70, 70))
    P = lambda b: C.c_uint64(b.ptr if b is not None else 0)
    for nh, nkv, hd, pos0, ntok in shapes:
        f = lambda *sh: (rng.standard_normal(sh) * 1.5).astype(np.float32)
        nctx = pos0 + ntok
        q, kc, vc = (hip.hip_upload_new(dev, a) for a in (f(ntok, nh * hd), f(nctx, nkv * hd), f(nctx, nkv * hd)))
        scratch = hip.hip_alloc(dev, 4 * ntok * nh * ((nctx + 3) & ~3))
        ints = (C.c_int(nh), C.c_int(nkv), C.c_int(hd), C.c_int(pos0), C.c_int(ntok))
        outs = []
        for scr in (None, scratch):
            out = hip.hip_upload_new(dev, np.full(ntok * nh * hd, np.nan, np.float32))
            hip.call("ilt_attn_rows", C.c_uint64(0), P(q), P(kc), P(vc), P(out), *ints, P(scr))
            outs.append(hip.hip_floats(out, ntok * nh * hd))
            hip.hip_free(out)
        assert np.array_equal(bits(outs[1]), bits(outs[0])), (nh, nkv, hd, pos0, ntok)
        for b in (q, kc, vc, scratch):
            hip.hip_free(b)


def test_decode_across_position_8192(dev):
    """A context longer than the 8,192 positions the kernels with their scores in memory take: tokens at positions 8,190
    and 8,191 go through ilt_dense_decode (tiled values), those at 8,192 and 8,193 through qk_rope + attn_rows with the
    scores in LDS, all with the oracle's logits bit for bit.  The caches' first 8,190 rows are filled with the same
    random keys and values on both sides instead of running a prompt that long through the oracle."""
    from illatio_amd import hip, model
    host = model.synth_model(61, d=256, ffn=512, nh=4, nkv=2, hd=64, nl=2, vocab=300)
    c = host["config"]
    nctx, pos0, kvd = 8200, 8190, c["nkv"] * c["hd"]
    rng = synth.make_rng(61)
    cpu = orc.DenseModel(host, nctx)
    gpu = model.DenseModel(dev, host, nctx, chunk=16)
    for li in range(c["nl"]):
        k, v = synth.activations((pos0, kvd), rng), synth.activations((pos0, kvd), rng)
        cpu.kc[li, :pos0], cpu.vc[li, :pos0] = k, v
        hip.hip_upload_vector(gpu.layers[li]["kc"], k)
        hip.hip_upload_vector(gpu.layers[li]["vc"], v)
    cpu.pos = gpu.pos = pos0
    tok = 17
    for step in range(4):
        want, _ = cpu.forward(tok, nthreads=16)
        gpu.forward_n([tok])
        got = hip.hip_floats(gpu.logits, c["vocab"])
        assert np.array_equal(bits(got), bits(want)), (pos0 + step, np.abs(got - want).max())
        tok = int(np.argmax(want))
    assert gpu.pos == 8194
    # a chunk that ends past 8,192 positions: the same fallback, the caches' rows as decode leaves them
    cpu2, gpu2 = orc.DenseModel(host, nctx), model.DenseModel(dev, host, nctx, chunk=16)
    for li in range(c["nl"]):
        cpu2.kc[li, :pos0], cpu2.vc[li, :pos0] = cpu.kc[li, :pos0], cpu.vc[li, :pos0]
        hip.hip_upload_vector(gpu2.layers[li]["kc"], cpu.kc[li, :pos0])
        hip.hip_upload_vector(gpu2.layers[li]["vc"], cpu.vc[li, :pos0])
    cpu2.pos = gpu2.pos = pos0
    toks = [5, 6, 7, 8, 9]
    for t in toks[:-1]:
        cpu2.forward(t, logits=False, nthreads=16)
    want, _ = cpu2.forward(toks[-1], nthreads=16)
    gpu2.forward_n(toks)
    assert np.array_equal(bits(hip.hip_floats(gpu2.logits, c["vocab"])), bits(want))
    with pytest.raises(ValueError):
        gpu2.forward_n([1] * 6)                                # past the context's 8,200 rows
    gpu.free(); gpu2.free()


def test_one_launch_attention_up_to_1024_positions(dev):
    """A token's attention in one launch (contexts of up to 1,024 positions, heads of 64 and of 128): decode steps in
    every one of its four blocks of 256 positions, on the blocks' edges, and across position 1023 -> 1024, where the
    two launches take over."""
    from illatio_amd import model
    for seed, hd, nh, nkv in ((21, 64, 4, 2), (22, 128, 4, 1)):
        host = model.synth_model(seed, d=256, ffn=512, nh=nh, nkv=nkv, hd=hd, nl=2, vocab=500)
        for nprompt, ndecode in ((250, 10), (508, 8), (764, 8), (1018, 10)):
            same, _ = run_greedy(dev, host, nprompt=nprompt, ndecode=ndecode, chunk=512, nctx=nprompt + ndecode + 2, seed=seed + nprompt)
            assert same == ndecode


def test_one_launch_attention_scores_shared_out(dev, monkeypatch):
    """The one-launch attention with a head's scores shared out over its workgroups (eight query heads: a head's
    workgroups then run on one die and exchange their scores inside the launch), in each block of 256 positions; the same
    with every workgroup giving up the wait at once and taking all the scores itself, and with the sharing switched off."""
    from illatio_amd import model
    for seed, hd, nkv in ((41, 64, 2), (42, 128, 4)):
        host = model.synth_model(seed, d=256, ffn=512, nh=8, nkv=nkv, hd=hd, nl=2, vocab=500)
        for mode in (None, "2", "0"):
            if mode is None:
                monkeypatch.delenv("ILT_ATTN_SPLIT", raising=False)
            else:
                monkeypatch.setenv("ILT_ATTN_SPLIT", mode)
            before = _giveups()
            for nprompt, ndecode in ((70, 6), (250, 10), (764, 6), (1018, 8)) if mode is None else ((250, 10), (1018, 8)):
                same, _ = run_greedy(dev, host, nprompt=nprompt, ndecode=ndecode, chunk=512, nctx=nprompt + ndecode + 2, seed=seed + nprompt)
                assert same == ndecode, (hd, mode, nprompt)
            # the library counts the workgroups that gave an exchange up: none where a head's workgroups find each other
            # (a slowdown of 200 us a launch could otherwise hide behind correct results), every one of them where told to
            gave_up = _giveups() - before
            assert (gave_up == 0) if mode is None else (gave_up > 0) if mode == "2" else (gave_up == 0), (hd, mode, gave_up)


def _giveups():
    import ctypes as C
    from illatio_amd import hip
    n = C.c_uint64(0)
    hip.call("ilt_attn_giveups", C.byref(n))
    return n.value


def test_two_decoders_on_two_streams_do_not_make_each_other_give_up(dev):
    """Two decoders stepping at once on one GPU, each on a stream of its own: the one-launch attention's exchange goes
    through a buffer per stream, so neither gives an exchange up (each step would take 200 us longer if they did),
    and both decode the tokens they decode alone."""
    from illatio_amd import hip, model
    host = model.synth_model(51, d=256, ffn=512, nh=8, nkv=2, hd=64, nl=2, vocab=500)
    rng = synth.make_rng(51)
    prompt = rng.integers(0, 500, 300).tolist()
    alone = model.DenseModel(dev, host, 340)
    alone.eval_tokens(prompt)
    want = alone.decode_greedy(24)
    alone.free()
    import ctypes as C
    info = hip.DeviceInfo()
    hip.call("ilt_device_get_info", C.c_int(dev.index), C.byref(info))
    other = hip.Device(dev.index, info, hip.hip_stream_create(dev))
    a, b = model.DenseModel(dev, host, 340), model.DenseModel(other, host, 340)
    a.eval_tokens(prompt); b.eval_tokens(prompt)
    hip.hip_sync(dev); hip.hip_stream_sync(other.stream)
    before = _giveups()
    got_a, got_b = [], []
    for _ in range(24):                                       # a token of each queued before either is waited for
        ta, tb = a.argmax(), b.argmax()
        got_a.append(ta); got_b.append(tb)
        a.forward_n([ta]); b.forward_n([tb])
    hip.hip_sync(dev); hip.hip_stream_sync(other.stream)
    assert got_a == want and got_b == want
    assert _giveups() == before
    a.free(); b.free()


def test_config_2_width_four_layers_128_greedy_tokens(dev):
    """Config 2's layer at its full width (hidden 2560, intermediate 9728, 32 query and 8 KV heads of 128, vocabulary
    151936), four layers: a 64-token prompt through the prefill products, then 128 greedy tokens, each step's logits
    with the CPU path's bits and so its top-1 token."""
    from illatio_amd import model
    host = model.synth_model(4, nl=4)
    same, margins = run_greedy(dev, host, nprompt=64, ndecode=128, chunk=64, nctx=200, seed=4)
    assert same == 128
    assert min(margins) > 0                                   # the greedy token was never a tie


def test_config_2_all_36_layers(dev):
    """All 36 layers of config 2's shape: an 8-token prompt and 12 greedy tokens, bit for bit."""
    from illatio_amd import model
    host = model.synth_model(36)
    same, _ = run_greedy(dev, host, nprompt=8, ndecode=12, chunk=8, nctx=24, seed=5)
    assert same == 12


def test_config_2_as_stated_36_layers_512_token_prompt_128_greedy_tokens(dev, capsys):
    """Config 2 at its stated size under the oracle: all 36 layers at full width, the seeded prompt of 512 random token
    ids through the prefill products in chunks of 128, then 128 greedy tokens at contexts of 512 to 639 positions (the
    one-launch attention with a head's scores shared out), every step's logits the CPU path's bit for bit -- hence the
    same top-1 token at every step, without a near-tie allowance; the smallest margin between the two best logits is
    printed and must be positive.  (The oracle's 640 positions take two to three minutes on the host's cores: a line is
    printed every 64 positions.)"""
    from illatio_amd import model

    def say(msg):
        with capsys.disabled():
            print("  [config 2]", msg, flush=True)

    host = model.synth_model(2)
    same, margins = run_greedy(dev, host, nprompt=512, ndecode=128, chunk=128, nctx=640, seed=22, say=say)
    assert same == 128
    say(f"128 greedy tokens, smallest top-1 margin {min(margins):.4f}, median {float(np.median(margins)):.4f}")
    assert min(margins) > 0


def _logprobs(v):
    v = v.astype(np.float64)
    m = v.max()
    return v - (m + np.log(np.exp(v - m).sum()))


CHAOTIC = pytest.mark.skip(reason="on the default random-init model every layer rewrites the residual stream and the attention is sharp: "
                              "measured, a prompt's K rows are 0.25 % (rms) from the CPU path's in layer 0, 2-9 % in layers 1-2 and 17 % in "
                              "layer 3, the logits' top ten move by up to 4.7 in logprob within 16 greedy steps and the top-1 token differs "
                              "at a step where the CPU path's two best are 0.67 apart (four layers, head_scale 8: step 7, 18 apart).  Not the "
                              "bf16 roundings: any difference from the CPU path, however small, grows to the size of a Q8_K step within two "
                              "layers, because the CPU path re-quantizes its activations before every product and a perturbed input rounds "
                              "to other quants (rms sqrt(difference x step)); in this model nothing damps it afterwards")


@pytest.mark.parametrize("prefill,damped", [("bf16", True), ("bf16-resident", True), pytest.param("bf16", False, marks=CHAOTIC)])
def test_bf16_prefill_keeps_the_top_1_token_over_128_greedy_tokens(dev, prefill, damped, capsys):
    """The prompt through the bf16 matrix-core products (on the CPU path's own quantized activations, each Q8_K quant
    times its block scale rounded to bf16), then 128 greedy tokens through the exact decode products reading the
    caches that prefill left: all 36 layers at config 2's width.  The bar is the reference's for its GPU path against
    its CPU path (inspect/cuda-consistency-test.lisp:19-22, 40-47): at every step the top-1 token is the CPU path's, or
    the two candidates lie closer than 0.1 in logprob (a near-tie), and no logprob among the top ten moves by 0.3.
    Each step is fed the CPU path's token, so one step's difference does not hide the next ones'.
    DAMPED: a random-init model conditioned as a trained one is -- a layer adds a fraction of the residual stream
    (update_scale), the attention's scores are soft (attn_temp), the logits spread like a language model's (std 2.7
    instead of 86) -- since the bar is in logprob and was set on trained checkpoints."""
    from illatio_amd import hip, model
    kw = dict(head_scale=0.25, update_scale=0.005, attn_temp=0.3) if damped else {}
    host = model.synth_model(4, nl=36 if damped else 4, **kw)
    c = host["config"]
    nprompt, ndecode = 64, 128
    rng = synth.make_rng(4)
    prompt = rng.integers(0, c["vocab"], nprompt).tolist()
    cpu = orc.DenseModel(host, nprompt + ndecode + 8)
    for t in prompt[:-1]:
        cpu.forward(t, logits=False, nthreads=16)
    want, _ = cpu.forward(prompt[-1], nthreads=16)
    gpu = model.DenseModel(dev, host, nprompt + ndecode + 8, chunk=64, prefill=prefill)
    gpu.eval_tokens(prompt)
    worst, differ = 0.0, 0
    for step in range(ndecode + 1):
        got = hip.hip_floats(gpu.logits, c["vocab"])
        a, b = _logprobs(got), _logprobs(want)
        top = np.argsort(-a)[:10]
        worst = max(worst, float(np.abs(a[top] - b[top]).max()))
        ga, wa = int(np.argmax(got)), int(np.argmax(want))
        if ga != wa:
            differ += 1
            assert float(a[ga] - a[wa]) < 0.1, (step, float(a[ga] - a[wa]))
        assert worst < 0.3, (step, worst)
        if step == ndecode:
            break
        want, _ = cpu.forward(wa, nthreads=16)
        gpu.forward_n([wa])
        if step % 32 == 31:
            with capsys.disabled():
                print(f"  [{prefill} prefill] step {step + 1}: top-1 differs at {differ} steps so far, worst |dlogprob| {worst:.4f}", flush=True)
    gpu.free()
    with capsys.disabled():
        print(f"  [{prefill} prefill] {ndecode} greedy tokens: top-1 differs at {differ} steps (near-ties), worst |dlogprob| in the top ten {worst:.4f}",
              flush=True)
