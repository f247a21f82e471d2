"""The GGUF container: header, metadata, tensor directory -- the host side of the reference's
src/gguf.lisp (READ-GGUF :105-147, GGUF-TENSOR :149-151, tensor bytes :153-157), plus the
step from a tensor in a file to a matrix on the device (UPLOAD-GMAT, cuda-dense.lisp:75-100).

All integers little-endian.  The header and directory are parsed; tensor data stays on
disk and is memory-mapped one tensor at a time, so a model is never held twice in memory.
"""
import struct

import numpy as np

MAGIC = 0x46554747          # "GGUF"

# ggml type code -> (name, elements per block, bytes per block)   (gguf.lisp:31-44)
GGML_TYPES = {
    0: ("f32", 1, 4), 1: ("f16", 1, 2), 2: ("q4_0", 32, 18), 3: ("q4_1", 32, 20), 6: ("q5_0", 32, 22), 7: ("q5_1", 32, 24),
    8: ("q8_0", 32, 34), 9: ("q8_1", 32, 36), 10: ("q2_k", 256, 84), 11: ("q3_k", 256, 110), 12: ("q4_k", 256, 144),
    13: ("q5_k", 256, 176), 14: ("q6_k", 256, 210), 15: ("q8_k", 256, 292), 16: ("iq2_xxs", 256, 66), 17: ("iq2_xs", 256, 74),
    18: ("iq3_xxs", 256, 98), 19: ("iq1_s", 256, 50), 20: ("iq4_nl", 32, 18), 21: ("iq3_s", 256, 110), 22: ("iq2_s", 256, 82),
    23: ("iq4_xs", 256, 136), 24: ("i8", 1, 1), 25: ("i16", 1, 2), 26: ("i32", 1, 4), 27: ("i64", 1, 8), 28: ("f64", 1, 8),
    29: ("iq1_m", 256, 56), 30: ("bf16", 1, 2), 39: ("mxfp4", 32, 17),
}


class GgufError(ValueError):
    pass


class TensorInfo:
    """NAME, DIMS in ggml order (ne0 is the contiguous axis), TYPE (ggml type code), OFFSET
    relative to the data section."""
    __slots__ = ("name", "dims", "type", "offset")

    def __init__(self, name, dims, type_, offset):
        self.name, self.dims, self.type, self.offset = name, tuple(dims), type_, offset

    @property
    def type_name(self):
        return GGML_TYPES[self.type][0]

    def elements(self):
        n = 1
        for d in self.dims:
            n *= d
        return n

    def nbytes(self):
        _, block, nb = GGML_TYPES[self.type]
        return self.elements() // block * nb


class Gguf:
    def __init__(self, path):
        self.path, self.version, self.metadata, self.tensors, self.tensor_order = path, 0, {}, {}, []
        self.data_offset, self.alignment = 0, 32

    def meta(self, key, default=None):
        return self.metadata.get(key, default)


class _Reader:
    def __init__(self, f):
        self.f = f

    def take(self, n):
        b = self.f.read(n)
        if len(b) != n:
            raise GgufError("GGUF: unexpected end of file")
        return b

    def uint(self, n):
        return int.from_bytes(self.take(n), "little", signed=False)

    def sint(self, n):
        return int.from_bytes(self.take(n), "little", signed=True)

    def string(self):
        n = self.uint(8)
        return self.take(n).decode("utf-8", errors="replace")

    def value(self, t):
        if t in (0, 2, 4, 10):
            return self.uint({0: 1, 2: 2, 4: 4, 10: 8}[t])
        if t in (1, 3, 5, 11):
            return self.sint({1: 1, 3: 2, 5: 4, 11: 8}[t])
        if t == 6:
            return struct.unpack("<f", self.take(4))[0]
        if t == 7:
            return self.uint(1) != 0
        if t == 8:
            return self.string()
        if t == 9:
            et, n = self.uint(4), self.uint(8)
            return [self.value(et) for _ in range(n)]
        if t == 12:
            return struct.unpack("<d", self.take(8))[0]
        raise GgufError(f"GGUF: unknown metadata value type {t}")


def read_gguf(path):
    """The header, metadata and tensor directory of the GGUF file at PATH (READ-GGUF)."""
    with open(path, "rb") as f:
        r = _Reader(f)
        if r.uint(4) != MAGIC:
            raise GgufError(f"{path} is not a GGUF file")
        g = Gguf(path)
        g.version = r.uint(4)
        n_tensors, n_kv = r.uint(8), r.uint(8)
        if g.version not in (2, 3):
            raise GgufError(f"GGUF version {g.version} is not supported (2 and 3 are)")
        for _ in range(n_kv):
            key = r.string()
            g.metadata[key] = r.value(r.uint(4))
        g.alignment = g.meta("general.alignment", 32)
        for _ in range(n_tensors):
            name = r.string()
            nd = r.uint(4)
            dims = [r.uint(8) for _ in range(nd)]
            code = r.uint(4)
            if code not in GGML_TYPES:
                raise GgufError(f"GGUF: unknown ggml tensor type {code}")
            g.tensors[name] = TensorInfo(name, dims, code, r.uint(8))
            g.tensor_order.append(name)
        a, p = g.alignment, f.tell()
        g.data_offset = a * ((p + a - 1) // a)
    return g


def gguf_tensor(g, name, errorp=True):
    ti = g.tensors.get(name)
    if ti is None and errorp:
        raise GgufError(f"GGUF: no tensor named {name!r}")
    return ti


def tensor_bytes(g, ti):
    """The tensor's raw bytes as a read-only memory map (nothing is copied until it is used)."""
    n = ti.nbytes()
    m = np.memmap(g.path, dtype=np.uint8, mode="r", offset=g.data_offset + ti.offset, shape=(n,)) if n else np.zeros(0, np.uint8)
    if m.size != n:
        raise GgufError(f"GGUF: truncated tensor {ti.name}")
    return m


def upload_tensor(dev, g, name):
    """The 2-D tensor NAME of G as a matrix on DEV (UPLOAD-GMAT): rows = ne1, columns = ne0."""
    from . import dense
    ti = gguf_tensor(g, name)
    if len(ti.dims) != 2:
        raise GgufError(f"{name}: {len(ti.dims)} dimensions, a matrix has two")
    cols, rows = ti.dims
    return dense.upload_gmat(dev, name, ti.type, rows, cols, tensor_bytes(g, ti))


def expert_tensor(g, name):
    """(TensorInfo, bytes a row, rows an expert, cols, experts) of the 3-D expert tensor NAME, dims
    [cols, rows, experts] (EXPERT-TENSOR, ds4f.lisp:95-100): expert e's rows start e * rows * row bytes in."""
    ti = gguf_tensor(g, name)
    if len(ti.dims) != 3:
        raise GgufError(f"{name}: {len(ti.dims)} dimensions, an expert tensor has three")
    cols, rows, ne = ti.dims
    return ti, ti.nbytes() // (rows * ne), rows, cols, ne


def upload_experts(dev, g, layer):
    """Layer LAYER's routed experts of G as an ExpertPool on DEV: blk.<layer>.ffn_gate_exps / ffn_up_exps
    (IQ2_XXS) and ffn_down_exps (Q2_K), each expert into its slot as gate | up | down (the slots D4-FILL
    makes, cuda-ds4f.lisp:162-166, 190-202; with all experts resident slot e is expert e)."""
    from . import ds4f
    from .synth import IQ2_XXS, Q2_K
    (gt, grb, ff, d, ne), (ut, urb, uff, ud, une), (dt, drb, dd, dff, dne) = (
        expert_tensor(g, f"blk.{layer}.ffn_{n}_exps.weight") for n in ("gate", "up", "down"))
    if (gt.type, ut.type, dt.type) != (IQ2_XXS, IQ2_XXS, Q2_K):
        raise GgufError(f"blk.{layer}: the expert products take IQ2_XXS gate/up and Q2_K down, not "
                        f"{gt.type_name}/{ut.type_name}/{dt.type_name}")
    if (uff, ud, une) != (ff, d, ne) or (dd, dff, dne) != (d, ff, ne):
        raise GgufError(f"blk.{layer}: the experts' gate, up and down do not fit one another")
    return ds4f.ExpertPool(dev, ne, d, ff, tensor_bytes(g, gt), tensor_bytes(g, ut), tensor_bytes(g, dt))


def upload_shared_expert(dev, g, layer):
    """Layer LAYER's shared expert (ffn_gate_shexp / ffn_up_shexp / ffn_down_shexp, Q8_0) repacked on DEV
    (D4-UPLOAD-WEIGHTS, cuda-ds4f.lisp:244-290)."""
    from . import ds4f
    from .synth import Q8_0
    tis = [gguf_tensor(g, f"blk.{layer}.ffn_{n}_shexp.weight") for n in ("gate", "up", "down")]
    for ti in tis:
        if ti.type != Q8_0 or len(ti.dims) != 2:
            raise GgufError(f"{ti.name}: the shared expert's matrices are 2-D Q8_0")
    d, ff = tis[0].dims
    if tuple(tis[1].dims) != (d, ff) or tuple(tis[2].dims) != (ff, d):
        raise GgufError(f"blk.{layer}: the shared expert's gate, up and down do not fit one another")
    return ds4f.SharedExpert(dev, d, ff, *(tensor_bytes(g, ti) for ti in tis))


DENSE_ARCHS = {"qwen2": True, "qwen3": True, "qwen3vl": True, "llama": False}       # architecture -> NEOX RoPE (model.lisp:94-96)


def dense_model(g):
    """The dense decoder in the GGUF file G as the dict illatio_amd.model.DenseModel takes (LOAD-MODEL-1,
    model.lisp:66-138): the architecture's keys into "config", every matrix as (GGUF type, its rows' bytes, memory-
    mapped), the norms and the attention biases (qwen2) as floats; without an output.weight the head is the embedding.
    Q8_0, Q4_K and Q6_K matrices (the decoder here multiplies those); anything else raises."""
    from .synth import Q4_K, Q6_K, Q8_0, row_bytes
    arch = g.meta("general.architecture")
    if arch not in DENSE_ARCHS:
        raise GgufError(f"architecture {arch!r} is not a dense decoder this loader reads ({', '.join(DENSE_ARCHS)} are)")
    key = lambda k, default=None: g.meta(f"{arch}.{k}", default)

    def need(k):
        v = key(k)
        if v is None:
            raise GgufError(f"GGUF: no {arch}.{k}")
        return v

    nl, d, nh = int(need("block_count")), int(need("embedding_length")), int(need("attention.head_count"))
    nkv = int(key("attention.head_count_kv", nh))
    hd = int(key("attention.key_length", d // nh))
    rd = int(key("rope.dimension_count", hd))
    if rd != hd:
        raise GgufError(f"RoPE over {rd} of a head's {hd} dimensions is not supported")

    def mat(name, rows, cols):
        ti = gguf_tensor(g, name)
        if ti.type not in (Q8_0, Q4_K, Q6_K):
            raise GgufError(f"{name}: type {ti.type_name}; the decoder here multiplies Q8_0, Q4_K and Q6_K matrices")
        if tuple(ti.dims) != (cols, rows):
            raise GgufError(f"{name}: dimensions {list(ti.dims)}, expected [{cols}, {rows}]")
        return ti.type, tensor_bytes(g, ti).reshape(rows, row_bytes(ti.type, cols))

    def f32(name, n, optional=False):
        ti = gguf_tensor(g, name, errorp=not optional)
        if ti is None:
            return None
        if GGML_TYPES[ti.type][0] != "f32" or ti.elements() != n:
            raise GgufError(f"{name}: expected {n} F32 values")
        return np.frombuffer(tensor_bytes(g, ti), np.float32).copy()

    ffn = int(need("feed_forward_length"))
    embd_ti = gguf_tensor(g, "token_embd.weight")
    vocab = int(embd_ti.dims[1])
    embd = mat("token_embd.weight", vocab, d)
    layers = []
    for i in range(nl):
        n = lambda t: f"blk.{i}.{t}"
        ffn_norm = f32(n("ffn_norm.weight"), d, optional=True)
        layers.append({"attn_norm": f32(n("attn_norm.weight"), d), "wq": mat(n("attn_q.weight"), nh * hd, d),
                       "wk": mat(n("attn_k.weight"), nkv * hd, d), "wv": mat(n("attn_v.weight"), nkv * hd, d),
                       "wo": mat(n("attn_output.weight"), d, nh * hd),
                       "bq": f32(n("attn_q.bias"), nh * hd, optional=True), "bk": f32(n("attn_k.bias"), nkv * hd, optional=True),
                       "bv": f32(n("attn_v.bias"), nkv * hd, optional=True),
                       "q_norm": f32(n("attn_q_norm.weight"), hd, optional=True), "k_norm": f32(n("attn_k_norm.weight"), hd, optional=True),
                       "ffn_norm": ffn_norm if ffn_norm is not None else f32(n("post_attention_norm.weight"), d),
                       "gate": mat(n("ffn_gate.weight"), ffn, d), "up": mat(n("ffn_up.weight"), ffn, d),
                       "down": mat(n("ffn_down.weight"), d, ffn)})
    output = mat("output.weight", vocab, d) if gguf_tensor(g, "output.weight", errorp=False) is not None else embd
    return {"config": {"d": d, "ffn": ffn, "nh": nh, "nkv": nkv, "hd": hd, "nl": nl, "vocab": vocab,
                       "eps": float(np.float32(need("attention.layer_norm_rms_epsilon"))), "rope_base": float(np.float32(key("rope.freq_base", 10000.0))),
                       "neox": DENSE_ARCHS[arch]},
            "embd": embd, "output": output, "output_norm": f32("output_norm.weight", d), "layers": layers}
