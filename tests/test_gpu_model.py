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


def run_greedy(dev, host, nprompt, ndecode, chunk, nctx, seed, check_cache=False):
    from illatio_amd import hip, model
    c = host["config"]
    rng = synth.make_rng(seed)
    prompt = rng.integers(0, c["vocab"], nprompt).tolist()
    cpu = orc.DenseModel(host, nctx)
    for t in prompt[:-1]:
        cpu.forward(t, logits=False, nthreads=16)
    want, _ = cpu.forward(prompt[-1], nthreads=16)
    gpu = model.DenseModel(dev, host, nctx, chunk=chunk)
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
    gpu.free()
    return same, margins


def test_small_decoder_prefill_chunks_and_decode(dev):
    from illatio_amd import model
    host = model.synth_model(3, d=512, ffn=1024, nh=8, nkv=2, hd=64, nl=3, vocab=1000)
    same, _ = run_greedy(dev, host, nprompt=40, ndecode=24, chunk=16, nctx=80, seed=1, check_cache=True)
    assert same == 24
    # a prompt of one token, and a chunk larger than the prompt
    run_greedy(dev, host, nprompt=1, ndecode=3, chunk=16, nctx=8, seed=2)
    run_greedy(dev, host, nprompt=9, ndecode=2, chunk=64, nctx=16, seed=3)


def test_small_decoder_long_contexts(dev):
    """Contexts past one workgroup's 256 positions of scores: the two-launch attention with 16 tokens, 4 tokens and one
    token a workgroup as the context grows towards 2048 positions, and past that the single launch with its value tiles."""
    from illatio_amd import model
    host = model.synth_model(6, d=256, ffn=512, nh=4, nkv=2, hd=64, nl=2, vocab=500)
    same, _ = run_greedy(dev, host, nprompt=2030, ndecode=6, chunk=512, nctx=2040, seed=6)
    assert same == 6
    same, _ = run_greedy(dev, host, nprompt=2060, ndecode=4, chunk=512, nctx=2100, seed=7)
    assert same == 4


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
