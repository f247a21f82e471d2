"""ilt_d4_ffn_step_noalloc, the entry point that allocates nothing: its output against
ilt_d4_ffn_step's (the same launches with the intermediates in a caller's workspace), bit
for bit, on two calls in a row of which the second is the smaller one -- the library's array
still holds the first call's contents then."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as orc
from illatio_amd import synth

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _layer(dev, rng, ne, d, ff):
    from illatio_amd import ds4f
    gate = synth.weights(synth.IQ2_XXS, ne * ff, d, rng)
    up = synth.weights(synth.IQ2_XXS, ne * ff, d, rng)
    down = synth.weights(synth.Q2_K, ne * d, ff, rng)
    sg, su = synth.weights(synth.Q8_0, ff, d, rng), synth.weights(synth.Q8_0, ff, d, rng)
    sd = synth.weights(synth.Q8_0, d, ff, rng)
    return (gate, up, down, sg, su, sd), ds4f.ExpertPool(dev, ne, d, ff, gate, up, down), ds4f.SharedExpert(dev, d, ff, sg, su, sd)


def test_no_alloc_step_equals_the_workspace_step_twice_in_a_row():
    from illatio_amd import ds4f, hip
    dev = hip.open_hip(0)
    rng = synth.make_rng(77)
    big = (12, 4096, 2048, 6, 0.0)            # config 4's step at a reduced expert count
    small = (8, 512, 256, 3, 0.05)
    layers = {shape: _layer(dev, rng, shape[0], shape[1], shape[2]) for shape in (big, small)}
    f = hip.lib().ilt_d4_ffn_step_noalloc_max_bytes
    f.restype = C.c_uint64
    assert f() == 1 << 20
    for ne, d, ff, nu, clamp in (big, small, big):          # the second call smaller than the first, then the large one again
        host, pool, sh = layers[(ne, d, ff, nu, clamp)]
        assert ds4f.step_workspace_bytes(nu, d, ff) <= f()
        logits, norm = synth.activations(ne, rng), synth.activations(d, rng)
        bias = (rng.standard_normal(ne) * 0.3).astype(np.float32)
        lb, nb, bb = hip.hip_upload_new(dev, logits), hip.hip_upload_new(dev, norm), hip.hip_upload_new(dev, bias)
        ref, out = hip.hip_alloc(dev, 4 * d), hip.hip_alloc(dev, 4 * d)
        for b in (None, bb):
            ds4f.ffn_step_call(dev, pool, sh, lb, nb, ref, ne, nu, 1.5, clamp, bias=b)
            ds4f.ffn_step_noalloc(dev, pool, sh, lb, nb, out, ne, nu, 1.5, clamp, bias=b)
            want, got = hip.hip_floats(ref, d), hip.hip_floats(out, d)
            assert np.array_equal(bits(got), bits(want)), (d, np.abs(got - want).max())
            cpu, _, _ = orc.moe_token(*host, d, ff, ne, nu, 1.5, clamp, logits, norm, bias=None if b is None else bias)
            assert np.array_equal(bits(got), bits(cpu))
            hip.hip_zero(out)
        for b in (lb, nb, bb, ref, out):
            hip.hip_free(b)
    # a step whose intermediates do not fit the array is refused, and nothing runs
    host, pool, sh = layers[small]
    lb, nb, out = hip.hip_upload_new(dev, np.zeros(8, np.float32)), hip.hip_upload_new(dev, np.zeros(512, np.float32)), hip.hip_alloc(dev, 4 * 512)
    pool.d, pool.ff, keep = 1 << 16, 1 << 16, (pool.d, pool.ff)            # 65536 x 65536 with 3 slots: 2.1 MB of intermediates
    pool.gate_bytes = pool.ff * (pool.d // 256 * 66)
    assert ds4f.step_workspace_bytes(3, pool.d, pool.ff) > f()
    with pytest.raises(hip.HipError):
        ds4f.ffn_step_noalloc(dev, pool, sh, lb, nb, out, 8, 3, 1.5, 0.0)
    pool.d, pool.ff = keep
    hip.hip_sync(dev)
    for b in (lb, nb, out):
        hip.hip_free(b)
    for _, pool, sh in layers.values():
        pool.free(); sh.free()
