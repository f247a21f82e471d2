"""The GGUF reader (illatio_amd/gguf.py ~ src/gguf.lisp) against files written by
tests/gguf_writer.py: metadata kinds, the tensor directory, alignment of the data section,
tensor sizes of the five block formats, the reference's error cases; and, on the GPU, a file's
tensors uploaded and multiplied with the oracle's bits."""
import struct

import numpy as np
import pytest

from illatio_amd import gguf, synth
from gguf_writer import write_gguf


def _tensors(rng):
    return [("blk.0.attn_q.weight", (512, 96), synth.Q4_K, synth.weights(synth.Q4_K, 96, 512, rng)),
            ("blk.0.attn_v.weight", (512, 40), synth.Q6_K, synth.weights(synth.Q6_K, 40, 512, rng)),
            ("blk.0.ffn_up.weight", (128, 72), synth.Q8_0, synth.weights(synth.Q8_0, 72, 128, rng)),
            ("blk.0.ffn_gate_exps.weight", (256, 16, 3), synth.IQ2_XXS, synth.weights(synth.IQ2_XXS, 48, 256, rng)),
            ("blk.0.ffn_down_exps.weight", (256, 8, 3), synth.Q2_K, synth.weights(synth.Q2_K, 24, 256, rng)),
            ("output_norm.weight", (512,), 0, np.arange(512, dtype=np.float32).view(np.uint8))]


@pytest.mark.parametrize("alignment", [None, 64, 4096])
def test_directory_metadata_and_bytes(tmp_path, alignment):
    rng = synth.make_rng(3)
    ts = _tensors(rng)
    md = {"general.architecture": "qwen3", "qwen3.block_count": 36, "qwen3.rope.freq_base": 1000000.0, "flag": True,
          "neg": -5, "tokenizer.ggml.tokens": ["a", "bc", "é"], "tokenizer.ggml.scores": [0.5, -1.0], "empty": []}
    p = tmp_path / "m.gguf"
    write_gguf(p, md, ts, alignment=alignment)
    g = gguf.read_gguf(str(p))
    assert g.version == 3 and g.alignment == (alignment or 32) and g.data_offset % g.alignment == 0
    assert g.meta("general.architecture") == "qwen3" and g.meta("qwen3.block_count") == 36 and g.meta("flag") is True
    assert g.meta("neg") == -5 and g.meta("tokenizer.ggml.tokens") == ["a", "bc", "é"] and g.meta("empty") == []
    assert g.meta("qwen3.rope.freq_base") == 1000000.0 and g.meta("missing", 7) == 7
    assert g.tensor_order == [t[0] for t in ts]
    for name, dims, code, raw in ts:
        ti = gguf.gguf_tensor(g, name)
        assert ti.dims == tuple(dims) and ti.type == code and ti.offset % g.alignment == 0
        assert ti.nbytes() == raw.size
        assert np.array_equal(np.asarray(gguf.tensor_bytes(g, ti)), raw.ravel())
    assert gguf.gguf_tensor(g, "nope", errorp=False) is None
    with pytest.raises(gguf.GgufError):
        gguf.gguf_tensor(g, "nope")


def test_block_sizes_are_ggml_s():
    for code, nbytes in ((8, 34), (10, 84), (12, 144), (14, 210), (16, 66)):
        assert gguf.GGML_TYPES[code][2] == nbytes == synth.BLOCK_BYTES[code]


def test_rejects_what_the_reference_rejects(tmp_path):
    p = tmp_path / "x.gguf"
    p.write_bytes(b"GGML" + b"\0" * 32)
    with pytest.raises(gguf.GgufError, match="not a GGUF file"):
        gguf.read_gguf(str(p))
    p.write_bytes(struct.pack("<IIQQ", gguf.MAGIC, 1, 0, 0))
    with pytest.raises(gguf.GgufError, match="version 1"):
        gguf.read_gguf(str(p))
    p.write_bytes(struct.pack("<IIQQ", gguf.MAGIC, 3, 1, 0) + struct.pack("<Q", 1) + b"t" + struct.pack("<IQIQ", 1, 32, 99, 0))
    with pytest.raises(gguf.GgufError, match="unknown ggml tensor type 99"):
        gguf.read_gguf(str(p))
    p.write_bytes(struct.pack("<IIQQ", gguf.MAGIC, 3, 0, 1) + struct.pack("<Q", 100) + b"short")
    with pytest.raises(gguf.GgufError, match="end of file"):
        gguf.read_gguf(str(p))
    write_gguf(p, {}, [("w", (256, 4), synth.Q4_K, synth.weights(synth.Q4_K, 4, 256, synth.make_rng(1)))])
    data = p.read_bytes()
    p.write_bytes(data[:-100])                     # the tensor's last bytes are missing
    g = gguf.read_gguf(str(p))
    with pytest.raises((gguf.GgufError, ValueError)):
        gguf.tensor_bytes(g, gguf.gguf_tensor(g, "w"))


def test_version_2_reads_like_3(tmp_path):
    p = tmp_path / "v2.gguf"
    write_gguf(p, {"k": 1}, [], version=2)
    g = gguf.read_gguf(str(p))
    assert g.version == 2 and g.meta("k") == 1 and g.tensor_order == []


@pytest.mark.gpu
def test_tensors_of_a_file_multiply_with_the_oracles_bits(tmp_path):
    import oracle_lib as orc
    from illatio_amd import dense, hip
    dev = hip.open_hip(0)
    rng = synth.make_rng(9)
    ts = _tensors(rng)
    p = tmp_path / "m.gguf"
    write_gguf(p, {"general.architecture": "test"}, ts, alignment=64)
    g = gguf.read_gguf(str(p))
    for name, dims, code, raw in ts[:3]:
        cols, rows = dims
        m = gguf.upload_tensor(dev, g, name)
        assert (m.rows, m.cols, m.type) == (rows, cols, code)
        x = synth.activations(cols, rng)
        xb, y = hip.hip_upload_new(dev, x), hip.hip_alloc(dev, 4 * rows)
        dense.mv_multi(dev, [(m, y, None)], xf=xb)
        want = orc.matmul(code, raw, rows, cols, x)
        assert np.array_equal(hip.hip_floats(y, rows).view(np.uint32), want.view(np.uint32))
        for b in (xb, y):
            hip.hip_free(b)
        m.free()
    with pytest.raises(gguf.GgufError):
        gguf.upload_tensor(dev, g, "output_norm.weight")


def _moe_file(tmp_path, rng, ne, d, ff):
    gate = synth.weights(synth.IQ2_XXS, ne * ff, d, rng)
    up = synth.weights(synth.IQ2_XXS, ne * ff, d, rng)
    down = synth.weights(synth.Q2_K, ne * d, ff, rng)
    sg, su, sd = synth.weights(synth.Q8_0, ff, d, rng), synth.weights(synth.Q8_0, ff, d, rng), synth.weights(synth.Q8_0, d, ff, rng)
    p = tmp_path / "moe.gguf"
    write_gguf(p, {"general.architecture": "deepseek4"}, [
        ("blk.3.ffn_gate_exps.weight", (d, ff, ne), synth.IQ2_XXS, gate), ("blk.3.ffn_up_exps.weight", (d, ff, ne), synth.IQ2_XXS, up),
        ("blk.3.ffn_down_exps.weight", (ff, d, ne), synth.Q2_K, down),
        ("blk.3.ffn_gate_shexp.weight", (d, ff), synth.Q8_0, sg), ("blk.3.ffn_up_shexp.weight", (d, ff), synth.Q8_0, su),
        ("blk.3.ffn_down_shexp.weight", (ff, d), synth.Q8_0, sd),
        ("blk.4.ffn_gate_exps.weight", (d, ff, ne), synth.Q4_K, synth.weights(synth.Q4_K, ne * ff, d, rng)),
        ("blk.4.ffn_up_exps.weight", (d, ff, ne), synth.IQ2_XXS, up), ("blk.4.ffn_down_exps.weight", (ff, d, ne), synth.Q2_K, down)])
    return p, (gate, up, down, sg, su, sd)


def test_expert_tensor_directory(tmp_path):
    """A 3-D expert tensor [cols, rows, experts]: bytes a row, rows an expert (EXPERT-TENSOR, ds4f.lisp:95-100)."""
    ne, d, ff = 5, 512, 256
    p, w = _moe_file(tmp_path, synth.make_rng(3), ne, d, ff)
    g = gguf.read_gguf(str(p))
    ti, rb, rows, cols, n = gguf.expert_tensor(g, "blk.3.ffn_gate_exps.weight")
    assert (rb, rows, cols, n) == (synth.row_bytes(synth.IQ2_XXS, d), ff, d, ne)
    ti, rb, rows, cols, n = gguf.expert_tensor(g, "blk.3.ffn_down_exps.weight")
    assert (rb, rows, cols, n) == (synth.row_bytes(synth.Q2_K, ff), d, ff, ne)
    raw = gguf.tensor_bytes(g, ti).reshape(ne, d * rb)
    assert np.array_equal(raw[4], w[2].reshape(ne, d * rb)[4])            # expert 4's rows start 4 * rows * row bytes in
    with pytest.raises(gguf.GgufError):
        gguf.expert_tensor(g, "blk.3.ffn_gate_shexp.weight")


@pytest.mark.gpu
def test_experts_of_a_file_take_a_decode_step_with_the_oracles_bits(tmp_path):
    """The routed experts (3-D tensors) and the shared expert of a written file, uploaded into slots and repacked
    (d4-upload-weights, cuda-ds4f.lisp:244-290), run one token's FFN with the CPU path's bits."""
    import oracle_lib as orc
    from illatio_amd import ds4f, hip
    dev = hip.open_hip(0)
    rng = synth.make_rng(12)
    ne, d, ff, nu = 6, 512, 256, 3
    p, (gate, up, down, sg, su, sd) = _moe_file(tmp_path, rng, ne, d, ff)
    g = gguf.read_gguf(str(p))
    pool, sh = gguf.upload_experts(dev, g, 3), gguf.upload_shared_expert(dev, g, 3)
    assert (pool.ne, pool.d, pool.ff, sh.d, sh.ff) == (ne, d, ff, d, ff)
    logits, norm = synth.activations(ne, rng), synth.activations(d, rng)
    want, _, _ = orc.moe_token(gate, up, down, sg, su, sd, d, ff, ne, nu, 1.5, 0.0, logits, norm)
    lb, nb, out = hip.hip_upload_new(dev, logits), hip.hip_upload_new(dev, norm), hip.hip_alloc(dev, 4 * d)
    ds4f.ffn_step_call(dev, pool, sh, lb, nb, out, ne, nu, 1.5, 0.0)
    assert np.array_equal(hip.hip_floats(out, d).view(np.uint32), want.view(np.uint32))
    with pytest.raises(gguf.GgufError, match="IQ2_XXS gate/up"):
        gguf.upload_experts(dev, g, 4)                                    # a Q4_K gate: not what the expert products take
    for b in (lb, nb, out):
        hip.hip_free(b)
    pool.free(); sh.free()


def _dense_file(tmp_path, host, arch="qwen3", tied=True):
    """HOST (model.synth_model's dict) as a GGUF file of architecture ARCH, as llama.cpp's converter names things."""
    c = host["config"]
    qd, kvd = c["nh"] * c["hd"], c["nkv"] * c["hd"]
    F32 = 0
    meta = {"general.architecture": arch, f"{arch}.block_count": c["nl"], f"{arch}.embedding_length": c["d"],
            f"{arch}.feed_forward_length": c["ffn"], f"{arch}.attention.head_count": c["nh"],
            f"{arch}.attention.head_count_kv": c["nkv"], f"{arch}.attention.key_length": c["hd"],
            f"{arch}.attention.layer_norm_rms_epsilon": float(c["eps"]), f"{arch}.rope.freq_base": float(c["rope_base"])}
    fb = lambda a: np.ascontiguousarray(a, np.float32).view(np.uint8)
    tensors = [("token_embd.weight", (c["d"], c["vocab"]), host["embd"][0], host["embd"][1]),
               ("output_norm.weight", (c["d"],), F32, fb(host["output_norm"]))]
    if not tied:
        tensors.append(("output.weight", (c["d"], c["vocab"]), host["output"][0], host["output"][1]))
    shapes = {"wq": ("attn_q", c["d"], qd), "wk": ("attn_k", c["d"], kvd), "wv": ("attn_v", c["d"], kvd), "wo": ("attn_output", qd, c["d"]),
              "gate": ("ffn_gate", c["d"], c["ffn"]), "up": ("ffn_up", c["d"], c["ffn"]), "down": ("ffn_down", c["ffn"], c["d"])}
    for i, L in enumerate(host["layers"]):
        for k, (name, cols, rows) in shapes.items():
            tensors.append((f"blk.{i}.{name}.weight", (cols, rows), L[k][0], L[k][1]))
        for k, name in (("attn_norm", "attn_norm.weight"), ("ffn_norm", "ffn_norm.weight"), ("q_norm", "attn_q_norm.weight"),
                        ("k_norm", "attn_k_norm.weight"), ("bq", "attn_q.bias"), ("bk", "attn_k.bias"), ("bv", "attn_v.bias")):
            if L.get(k) is not None:
                tensors.append((f"blk.{i}.{name}", (len(L[k]),), F32, fb(L[k])))
    p = tmp_path / f"{arch}.gguf"
    write_gguf(p, meta, tensors)
    return p


def test_dense_model_of_a_file(tmp_path):
    """gguf.dense_model (load-model-1, model.lisp:66-138): the architecture's keys, every matrix and norm of a written
    qwen3-style file, the head tied to the embedding when the file has no output.weight; files it does not read raise."""
    from illatio_amd import model
    host = model.synth_model(21, d=256, ffn=512, nh=4, nkv=2, hd=64, nl=2, vocab=300)
    g = gguf.read_gguf(str(_dense_file(tmp_path, host)))
    got = gguf.dense_model(g)
    f32 = lambda c: {k: (float(np.float32(v)) if isinstance(v, float) else v) for k, v in c.items()}      # the file holds singles
    assert f32(got["config"]) == f32(host["config"])
    assert got["output"] is got["embd"]
    assert got["embd"][0] == host["embd"][0] and np.array_equal(got["embd"][1], host["embd"][1])
    assert np.array_equal(got["output_norm"], host["output_norm"])
    def same_layers(got, host):
        for a, b in zip(got["layers"], host["layers"]):
            assert {k for k in a if a[k] is not None} == {k for k in b if b[k] is not None}
            for k in b:
                if isinstance(b[k], tuple):
                    assert a[k][0] == b[k][0] and np.array_equal(a[k][1], b[k][1]), k
                elif b[k] is not None:
                    assert np.array_equal(a[k], b[k]), k
    same_layers(got, host)
    # a qwen2-style file: Q8_0 matrices, biases on Q, K and V, no head norms
    hostq = model.synth_model_q8(23, d=256, ffn=512, nh=4, nkv=2, hd=64, nl=2, vocab=300)
    gotq = gguf.dense_model(gguf.read_gguf(str(_dense_file(tmp_path, hostq, arch="qwen2"))))
    assert gotq["layers"][0]["q_norm"] is None and gotq["layers"][0]["bq"] is not None and gotq["embd"][0] == synth.Q8_0
    same_layers(gotq, hostq)
    host2 = dict(host, output=(host["embd"][0], host["embd"][1][::-1].copy()))
    got2 = gguf.dense_model(gguf.read_gguf(str(_dense_file(tmp_path, host2, arch="llama", tied=False))))
    assert got2["config"]["neox"] is False and got2["output"] is not got2["embd"]
    assert np.array_equal(got2["output"][1], host2["output"][1])
    with pytest.raises(gguf.GgufError):
        gguf.dense_model(gguf.read_gguf(str(_dense_file(tmp_path, host, arch="deepseek4"))))
    bad = dict(host, layers=[dict(L, wq=(synth.Q2_K, synth.weights(synth.Q2_K, 256, 256, synth.make_rng(1)))) for L in host["layers"]])
    with pytest.raises(gguf.GgufError):
        gguf.dense_model(gguf.read_gguf(str(_dense_file(tmp_path, bad))))


@pytest.mark.gpu
@pytest.mark.parametrize("arch", ["qwen3", "qwen2"])
def test_decoder_of_a_file_decodes_with_the_oracles_bits(tmp_path, arch):
    """A written qwen3-style file (K-quants, head norms) and a qwen2-style one (Q8_0, biases) read back, uploaded and
    run: prompt and greedy tokens with the CPU oracle's logits."""
    import oracle_lib as orc
    from illatio_amd import hip, model
    dev = hip.open_hip(0)
    make = model.synth_model if arch == "qwen3" else model.synth_model_q8
    host = make(22, d=256, ffn=512, nh=4, nkv=2, hd=64, nl=2, vocab=300)
    got = gguf.dense_model(gguf.read_gguf(str(_dense_file(tmp_path, host, arch=arch))))
    cpu, gpu = orc.DenseModel(host, 24), model.DenseModel(dev, got, 24, chunk=8)
    prompt = [5, 17, 255, 3, 99, 100, 1, 42, 7, 8, 9]
    for t in prompt[:-1]:
        cpu.forward(t, logits=False, nthreads=4)
    want, _ = cpu.forward(prompt[-1], nthreads=4)
    gpu.eval_tokens(prompt)
    for _ in range(6):
        have = hip.hip_floats(gpu.logits, 300)
        assert np.array_equal(have.view(np.uint32), want.view(np.uint32))
        tok = int(np.argmax(want))
        want, _ = cpu.forward(tok, nthreads=4)
        gpu.forward_n([tok])
    gpu.free()
