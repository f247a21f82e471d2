"""A dense decoder on the device: the host side of the reference's CUDA-FORWARD-N (src/cuda-dense.lisp:380-432)
for the K-quant models of the benchmark's config 2 and the Q8_0 ones of config 1 (qwen2: biases on Q, K and V, no head
norms) -- embedding, and per layer: norm, Q/K/V, head norms + RoPE +
cache update, attention, wo added to the stream, norm, gate/up with swiglu!, down added to the stream; then the
output norm and head.  One token runs the decode products (matrix-vector kernels that take the norm and the
quantizer inside); several tokens run the prefill products (EVAL-TOKENS, batch.lisp:289-307).  Either way a
token's logits have the CPU path's bits (FORWARD-1, model.lisp:396-462): the products are bit-exact and the
kernels between them add in the CPU's order.

synth_model makes the random-init model the benchmark and the tests run (there are no model files here):
Q4_K for most matrices, Q6_K for V, down and the tied embedding / output head, as Q4_K_M files have them.
"""
import ctypes as C

import numpy as np

from . import dense, hip, synth
from .synth import Q4_K, Q6_K, Q8_0


def synth_model(seed, d=2560, ffn=9728, nh=32, nkv=8, hd=128, nl=36, vocab=151936, eps=1e-6, rope_base=1e6, head_scale=8.0, update_scale=1.0, attn_temp=1.0):
    """A seeded random-init dense decoder as numpy arrays: {"config", "embd", "output", "output_norm", "layers"}; a
    matrix is (GGUF type, uint8 rows).  HEAD_SCALE spreads the output head's logits so that the greedy token is not
    decided in the last bits (random weights give nearly flat logits).  UPDATE_SCALE multiplies the block scales of wo
    and down, i.e. what a layer adds to the residual stream: at 1 a layer's update is some forty times the stream it
    is added to, so every layer rewrites the stream (the hardest case for bit-exactness, and one where any rounding
    difference grows about fivefold a layer); around 0.005 the stream dominates its updates, as in a trained model.  ATTN_TEMP multiplies the query heads' norm weights, i.e.
    the attention's scores (at 1 they are about N(0, 1)).  Neither changes the values drawn at 1."""
    rng = synth.make_rng(seed)
    qd, kvd = nh * hd, nkv * hd
    if d % 256 or qd % 256 or ffn % 256:
        raise ValueError("K-quant rows are whole super-blocks of 256 columns: d, nh * hd and ffn must be multiples of 256")
    norm = lambda n: (synth.activations(n, rng) * 0.1 + 1.0).astype(np.float32)
    layers = []
    for _ in range(nl):
        layers.append({"wq": (Q4_K, synth.weights(Q4_K, qd, d, rng)), "wk": (Q4_K, synth.weights(Q4_K, kvd, d, rng)),
                       "wv": (Q6_K, synth.weights(Q6_K, kvd, d, rng)), "wo": (Q4_K, synth.weights(Q4_K, d, qd, rng, dscale=0.0002 * update_scale)),
                       "gate": (Q4_K, synth.weights(Q4_K, ffn, d, rng)), "up": (Q4_K, synth.weights(Q4_K, ffn, d, rng)),
                       "down": (Q6_K, synth.weights(Q6_K, d, ffn, rng, dscale=0.002 / 32.0 * update_scale)),
                       "attn_norm": norm(d), "ffn_norm": norm(d), "q_norm": (norm(hd) * attn_temp).astype(np.float32), "k_norm": norm(hd)})
    embd = (Q6_K, synth.weights(Q6_K, vocab, d, rng, dscale=0.01 * head_scale / 32.0))
    return {"config": {"d": d, "ffn": ffn, "nh": nh, "nkv": nkv, "hd": hd, "nl": nl, "vocab": vocab, "eps": eps, "rope_base": rope_base,
                       "neox": True},
            "embd": embd, "output": embd, "output_norm": norm(d), "layers": layers}


def synth_model_q8(seed, d=896, ffn=4864, nh=14, nkv=2, hd=64, nl=24, vocab=151936, eps=1e-6, rope_base=1e6, head_scale=8.0):
    """The same for the benchmark's config 1 family (Qwen2.5-0.5B in Q8_0): every matrix Q8_0, biases on Q, K and V,
    no head norms, the head tied to the embedding."""
    rng = synth.make_rng(seed)
    qd, kvd = nh * hd, nkv * hd
    norm = lambda n: (synth.activations(n, rng) * 0.1 + 1.0).astype(np.float32)
    bias = lambda n: (synth.activations(n, rng) * 0.5).astype(np.float32)
    q8 = lambda rows, cols: (Q8_0, synth.weights(Q8_0, rows, cols, rng))
    layers = [{"wq": q8(qd, d), "wk": q8(kvd, d), "wv": q8(kvd, d), "wo": q8(d, qd), "gate": q8(ffn, d), "up": q8(ffn, d), "down": q8(d, ffn),
               "bq": bias(qd), "bk": bias(kvd), "bv": bias(kvd), "attn_norm": norm(d), "ffn_norm": norm(d), "q_norm": None, "k_norm": None}
              for _ in range(nl)]
    embd = q8(vocab, d)
    return {"config": {"d": d, "ffn": ffn, "nh": nh, "nkv": nkv, "hd": hd, "nl": nl, "vocab": vocab, "eps": eps, "rope_base": rope_base,
                       "neox": True},
            "embd": embd, "output": embd, "output_norm": norm(d), "layers": layers}


class _Mat(C.Structure):
    _fields_ = [("gguf_type", C.c_int), ("rows", C.c_int), ("cols", C.c_int), ("w", C.c_uint64), ("wd", C.c_uint64)]


class _Layer(C.Structure):
    _fields_ = [("attn_norm", C.c_uint64), ("q_norm", C.c_uint64), ("k_norm", C.c_uint64), ("ffn_norm", C.c_uint64)] + \
               [(n, _Mat) for n in ("wq", "wk", "wv", "wo", "gate", "up", "down")] + [("kc", C.c_uint64), ("vc", C.c_uint64)] + \
               [(n, C.c_uint64) for n in ("bq", "bk", "bv")]


class _Model(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("nl", "d", "ffn", "nh", "nkv", "hd", "rd", "neox", "nctx")] + [("eps", C.c_float), ("embd", _Mat), ("output", _Mat),
               ("output_norm", C.c_uint64), ("rope", C.c_uint64), ("layers", C.POINTER(_Layer))] + \
               [(n, C.c_uint64) for n in ("x", "q", "k", "v", "att", "fa", "scores", "logits")]


def _mat(w):
    return _Mat(w.type, w.rows, w.cols, w.qs.ptr, w.d.ptr if w.d else 0)


PARTS_WORK = 1e10
PARTS_FROM, PARTS_UPTO = 256, 4096      # eval_tokens: chunks of so many tokens as parts side by side on streams of their own (0, -1: never)


class _Work:
    """A chunk's buffers and the device handle (its stream) their launches go to."""


class DenseModel:
    """HOST (synth_model's dict, or the same made from a file's tensors) on DEV, with caches for NCTX positions."""

    def __init__(self, dev, host, nctx, chunk=2048, prefill="exact"):
        """CHUNK: the tokens of a prompt that go through the layers together (*CUDA-CHUNK*, cuda-dense.lisp:29, is 512;
        on 256 CUs a 512-token chunk's smaller products -- V, wo, down -- are 64 to 160 workgroups, and a 2,048-token
        prompt takes 79.6 ms in one chunk against 99.1 ms in four; the results do not depend on it).
        PREFILL: how a chunk of several tokens is multiplied.  "exact": the int8 products, every token with the bits
        of its own decode step (the CPU path's MATMUL!).  "bf16": the bf16 matrix-core products on the CPU path's own
        quantized activations (each Q8_K quant times its block scale, rounded to bf16), K-quant matrices only: within
        the bf16 roundings of the exact products, not equal to them.  "bf16-resident": the same numbers from bf16
        copies of the matrices made once here and kept beside the quantized ones that decode reads (2 bytes a
        weight).  One token always takes the decode products."""
        c = host["config"]
        if prefill not in ("exact", "bf16", "bf16-resident"):
            raise ValueError(f"prefill {prefill!r}: exact, bf16 or bf16-resident")
        self.prefill = prefill
        chunk = max(1, min(chunk, nctx))
        self.dev, self.c, self.nctx, self.chunk, self.pos = dev, c, nctx, chunk, 0
        d, ffn, hd = c["d"], c["ffn"], c["hd"]
        self.qd, self.kvd = c["nh"] * hd, c["nkv"] * hd
        up = lambda name, m, rows, cols: dense.upload_gmat(dev, name, m[0], rows, cols, m[1])
        fl = lambda a: None if a is None else hip.hip_upload_new(dev, np.ascontiguousarray(a, np.float32))
        self.layers = []
        for li, L in enumerate(host["layers"]):
            self.layers.append({"wq": up(f"blk.{li}.attn_q", L["wq"], self.qd, d), "wk": up(f"blk.{li}.attn_k", L["wk"], self.kvd, d),
                                "wv": up(f"blk.{li}.attn_v", L["wv"], self.kvd, d), "wo": up(f"blk.{li}.attn_output", L["wo"], d, self.qd),
                                "gate": up(f"blk.{li}.ffn_gate", L["gate"], ffn, d), "up": up(f"blk.{li}.ffn_up", L["up"], ffn, d),
                                "down": up(f"blk.{li}.ffn_down", L["down"], d, ffn),
                                "attn_norm": fl(L["attn_norm"]), "ffn_norm": fl(L["ffn_norm"]), "q_norm": fl(L.get("q_norm")),
                                "k_norm": fl(L.get("k_norm")), "bq": fl(L.get("bq")), "bk": fl(L.get("bk")), "bv": fl(L.get("bv")),
                                "kc": hip.hip_alloc(dev, 4 * nctx * self.kvd), "vc": hip.hip_alloc(dev, 4 * nctx * self.kvd)})
        self.embd = up("token_embd", host["embd"], c["vocab"], d)
        self.output = self.embd if host["output"] is host["embd"] else up("output", host["output"], c["vocab"], d)
        self.output_norm = fl(host["output_norm"])
        rope = np.empty((nctx, hd), np.float32)
        hip.call("ilt_rope_table", C.c_int(hd), C.c_int(0), C.c_int(nctx), C.c_float(c["rope_base"]), rope.ctypes.data_as(C.c_void_p))
        self.rope = hip.hip_upload_new(dev, rope)
        self.logits = hip.hip_alloc(dev, 4 * c["vocab"])
        # a chunk's quantized activations per width, in the formats the matrices that read that width take
        # (Q8_0 blocks for Q8_0 matrices, Q8_K blocks for K-quants, as the CPU path makes them)
        reads = {d: ("wq", "wk", "wv", "gate", "up"), self.qd: ("wo",), ffn: ("down",)}
        self._kinds = {}
        for cols, names in reads.items():
            for L in self.layers:
                for nm in names:
                    self._kinds.setdefault(cols, set()).add("q8k" if L[nm].kquant_p() else "q8")
        if prefill != "exact" and any("q8" in k for k in self._kinds.values()):
            raise ValueError("the bf16 prefill multiplies K-quant matrices; this model has Q8_0 ones")
        # the buffers a chunk goes through the layers in (more sets, each on a stream of its own, are made when the
        # parts of a chunk first go side by side: eval_tokens)
        self.work, self.more_work, self._keys_ev, self._join_ev = self._work_set(dev, chunk), [], [], []
        w = self.work
        self.x, self.q, self.k, self.v, self.att, self.fa, self.fb = w.x, w.q, w.k, w.v, w.att, w.fa, w.fb
        self.tokens, self.scores, self.acts, self.xb = w.tokens, w.scores, w.acts, w.xb
        self.wb = {}
        if prefill != "exact":
            if prefill == "bf16-resident":
                for li, L in enumerate(self.layers):
                    for nm in ("wq", "wk", "wv", "wo", "gate", "up", "down"):
                        self.wb[(li, nm)] = dense.dequant_bf16(dev, L[nm])
        # the model as ilt_dense_decode reads it: a token's launches queued by one call
        ptr = lambda b: b.ptr if b is not None else 0
        self._clayers = (_Layer * len(self.layers))()
        for i, L in enumerate(self.layers):
            self._clayers[i] = _Layer(ptr(L["attn_norm"]), ptr(L["q_norm"]), ptr(L["k_norm"]), ptr(L["ffn_norm"]),
                                      *[_mat(L[n]) for n in ("wq", "wk", "wv", "wo", "gate", "up", "down")], L["kc"].ptr, L["vc"].ptr,
                                      ptr(L["bq"]), ptr(L["bk"]), ptr(L["bv"]))
        self._cmodel = _Model(len(self.layers), d, ffn, c["nh"], c["nkv"], hd, hd, 1 if c["neox"] else 0, nctx, c["eps"], _mat(self.embd), _mat(self.output),
                              self.output_norm.ptr, self.rope.ptr, self._clayers, self.x.ptr, self.q.ptr, self.k.ptr, self.v.ptr, self.att.ptr,
                              self.fa.ptr, ptr(self.scores), self.logits.ptr)
        self.one_call = True                          # False: a token's launches one by one from here (the same launches)

    def _work_set(self, dev, n):
        """The buffers N tokens go through the layers in, their launches on DEV's stream."""
        c = self.c
        d, ffn = c["d"], c["ffn"]
        A = lambda nbytes: hip.hip_alloc(dev, nbytes)
        w = _Work()
        w.dev, w.n = dev, n
        w.x, w.q, w.k, w.v = A(4 * n * d), A(4 * n * self.qd), A(4 * n * self.kvd), A(4 * n * self.kvd)
        w.att, w.fa, w.fb = A(4 * n * self.qd), A(4 * n * ffn), A(4 * n * ffn)
        w.tokens = A(4 * n)
        # the attention's raw scores, for the positions the kernels that keep them in memory take (up to 8192); past
        # those a token's attention runs as one launch with its scores in LDS
        w.scores = A(4 * n * c["nh"] * ((min(self.nctx, 8192) + 3) // 4 * 4))
        w.acts = {cols: dense.QAct(dev, n, cols, tuple(sorted(k))) for cols, k in self._kinds.items()}
        # a chunk's activations as bf16 per width (rows, or slabs for the resident copies' product)
        w.xb = {} if self.prefill == "exact" else {cols: hip.hip_alloc(dev, dense.slabs_bytes(n, cols), zero=False) for cols in self._kinds}
        return w

    def _free_work(self, w):
        for b in (w.x, w.q, w.k, w.v, w.att, w.fa, w.fb, w.tokens, w.scores):
            hip.hip_free(b)
        for a in w.acts.values():
            a.free()
        for b in w.xb.values():
            hip.hip_free(b)

    def forward_n(self, tokens, logits=True):
        """TOKENS at the next positions (CUDA-FORWARD-N); the last one's logits, if LOGITS, into self.logits."""
        n = len(tokens)
        if n < 1 or n > self.chunk or self.pos + n > self.nctx:
            raise ValueError(f"{n} tokens at position {self.pos}: the chunk holds {self.chunk}, the context {self.nctx}")
        for _ in self._steps(tokens, self.pos, logits, self.work):
            pass
        self.pos += n
        return self.logits

    def _steps(self, tokens, pos, logits, W):
        """forward_n's launches for TOKENS at positions POS.. in the work set W, as a generator: it yields ("keys", layer)
        when a layer's keys and values are queued for the caches and ("layer", layer) when the layer is."""
        dev, c, n = W.dev, self.c, len(tokens)
        d, ffn, hd, nh, nkv, eps = c["d"], c["ffn"], c["hd"], c["nh"], c["nkv"], c["eps"]
        S = C.c_uint64(dev.stream)
        P = lambda b, off=0: C.c_uint64(b.ptr + off if b is not None else 0)
        hip.hip_upload_vector(W.tokens, np.asarray(tokens, np.int32))
        scratch = W.scores if pos + n <= 8192 else None
        if n == 1 and self.one_call and scratch is not None and W is self.work:
            hip.call("ilt_dense_decode", S, C.byref(self._cmodel), P(W.tokens), C.c_int(pos), C.c_int(1 if logits else 0))
            return
        dense.embed(dev, self.embd, W.tokens, W.x, n, d)
        fast = self.prefill != "exact" and n > 1
        slabs = self.prefill == "bf16-resident"

        def mul_fast(li, parts, act, acc=False):
            """PARTS (name, y, bias) on ACT's Q8_K blocks taken as bf16."""
            xb = dense.q8k_bf16(dev, act, n, out=W.xb[act.cols], slabs=slabs)

            def run(nm, y, bias):
                w = self.layers[li][nm]
                if slabs:
                    dense.mat_mul_bf16(dev, self.wb[(li, nm)], w.rows, w.cols, xb, y, n, bias=bias, acc=acc)
                else:
                    dense.cmat_mul_bf16(dev, w, xb, y, n, bias=bias, acc=acc)

            # the products after the first on the device's second stream (not the resident copies': 256 x 256 tiles, a
            # workgroup a CU, and two launches at once were 3.5 % slower than one after the other)
            if len(parts) > 1 and dense.BESIDE and not slabs:
                with hip.beside(dev):
                    for pt in parts[1:]:
                        run(*pt)
                run(*parts[0])
                hip.rejoin(dev)
            else:
                for pt in parts:
                    run(*pt)

        def gated():
            """The chunk's gated activations as the down product reads them: swiglu and the quantizer in one launch, or
            (a model with Q8_0 matrices) one after the other."""
            a = dense.swiglu_quantize_act(dev, W.fa, W.fb, W.acts[ffn], n)
            if a is None:
                hip.call("ilt_swiglu", S, P(W.fa), P(W.fb), C.c_int64(n * ffn))
                a = dense.quantize_act(dev, W.fa, W.acts[ffn], n=n)
            return a

        for li, L in enumerate(self.layers):
            if n == 1:
                dense.qkv_mul(dev, L["wq"], L["wk"], L["wv"], None, W.q, W.k, W.v, L["bq"], L["bk"], L["bv"], xf=W.x,
                              norm=(L["attn_norm"], eps))
            else:
                a = dense.rmsnorm_q8(dev, W.x, L["attn_norm"], W.acts[d], d, eps, n=n)
                if fast:
                    mul_fast(li, [("wq", W.q, L["bq"]), ("wk", W.k, L["bk"]), ("wv", W.v, L["bv"])], a)
                else:
                    dense.cmat_mul_n(dev, [(L["wq"], W.q, L["bq"]), (L["wk"], W.k, L["bk"]), (L["wv"], W.v, L["bv"])], a, n)
            if n == 1 and scratch is not None:
                hip.call("ilt_attn_step", S, P(W.q), P(W.k), P(W.v), P(L["q_norm"]), P(L["k_norm"]), P(self.rope), P(L["kc"]), P(L["vc"]),
                         P(W.att), C.c_int(nh), C.c_int(nkv), C.c_int(hd), C.c_int(hd), C.c_int(pos), C.c_float(eps),
                         C.c_int(1 if c["neox"] else 0), P(W.scores), C.c_int(self.nctx))
            else:
                hip.call("ilt_qk_rope", S, P(W.q), P(W.k), P(W.v), P(L["q_norm"]), P(L["k_norm"]), P(self.rope), P(L["kc"]), P(L["vc"]),
                         C.c_int(nh), C.c_int(nkv), C.c_int(hd), C.c_int(hd), C.c_int(pos), C.c_float(eps), C.c_int(1 if c["neox"] else 0),
                         C.c_int(n))
                yield ("keys", li)
                hip.call("ilt_attn_rows", S, P(W.q), P(L["kc"]), P(L["vc"]), P(W.att), C.c_int(nh), C.c_int(nkv), C.c_int(hd),
                         C.c_int(pos), C.c_int(n), P(scratch))
            if n == 1:
                dense.mv_multi(dev, [(L["wo"], W.x, None)], xf=W.att, acc=True)
                dense.glu_mul(dev, L["gate"], L["up"], None, W.fa, xf=W.x, norm=(L["ffn_norm"], eps))
                dense.mv_multi(dev, [(L["down"], W.x, None)], xf=W.fa, acc=True)
            elif fast:
                mul_fast(li, [("wo", W.x, None)], dense.quantize_act(dev, W.att, W.acts[self.qd], n=n), acc=True)
                mul_fast(li, [("gate", W.fa, None), ("up", W.fb, None)], dense.rmsnorm_q8(dev, W.x, L["ffn_norm"], W.acts[d], d, eps, n=n))
                mul_fast(li, [("down", W.x, None)], gated(), acc=True)
            else:
                dense.cmat_mul(dev, L["wo"], dense.quantize_act(dev, W.att, W.acts[self.qd], n=n), W.x, n=n, acc=True)
                a = dense.rmsnorm_q8(dev, W.x, L["ffn_norm"], W.acts[d], d, eps, n=n)
                dense.cmat_mul_n(dev, [(L["gate"], W.fa, None), (L["up"], W.fb, None)], a, n)
                dense.cmat_mul(dev, L["down"], gated(), W.x, n=n, acc=True)
            yield ("layer", li)
        if logits:
            last = hip.DBuf(W.x.ptr + 4 * (n - 1) * d, 4 * d, dev)
            dense.mv_multi(dev, [(self.output, self.logits, None)], xf=last, norm=(self.output_norm, eps))

    def decode_greedy(self, ntokens):
        """NTOKENS greedy tokens after what the context holds, the first one picked from self.logits: every token picked
        on the device (ilt_argmax) and fed to the next step from device memory, nothing waited for until the ids are
        read back at the end.  Returns the ids; self.logits holds the logits after the last of them."""
        if not self.one_call or self.pos + ntokens > 8192:
            raise ValueError("the device-side loop runs over ilt_dense_decode (contexts up to 8192 positions)")
        if self.pos + ntokens > self.nctx:
            raise ValueError(f"{ntokens} more tokens at position {self.pos}: the context holds {self.nctx}")
        dev, vocab = self.dev, self.c["vocab"]
        S = C.c_uint64(dev.stream)
        ids, scratch = hip.hip_alloc(dev, 4 * ntokens), hip.hip_alloc(dev, 2048)
        for i in range(ntokens):
            hip.call("ilt_argmax", S, C.c_uint64(self.logits.ptr), C.c_int(vocab), C.c_uint64(ids.ptr + 4 * i), C.c_uint64(scratch.ptr))
            hip.call("ilt_dense_decode", S, C.byref(self._cmodel), C.c_uint64(ids.ptr + 4 * i), C.c_int(self.pos), C.c_int(1))
            self.pos += 1
        out = hip.hip_download(ids, np.int32, ntokens).tolist()
        hip.hip_free(ids)
        hip.hip_free(scratch)
        return out

    def reset(self):
        """Forget the tokens seen: the next one is at position 0 (the caches' rows are overwritten as positions are reached)."""
        self.pos = 0

    def forward_parts(self, tokens, logits=True, k=2):
        """forward_n with TOKENS as K parts side by side, each in buffers and on a stream of its own, every part a step
        behind the one before it: its attention in a layer waits for the earlier parts' keys and values of that layer
        (an event each), and nothing else of one part depends on another.  A chunk of a few hundred tokens leaves
        most of its launches with fewer workgroups than the GPU has room for (at 512 tokens V is 64 workgroups, wo and
        down 160, of 512 that fit), and while one part is in its attention (vector ALU) another is in its products
        (matrix cores): the parts' launches fill each other's gaps.  Every token's results are forward_n's."""
        n, dev = len(tokens), self.dev
        per = ((n + k - 1) // k + 127) // 128 * 128
        if k < 2 or per * (k - 1) >= n or n > self.chunk or self.pos + n > self.nctx or self.pos + n > 8192:
            return self.forward_n(tokens, logits)
        while len(self.more_work) < k - 1:
            import copy
            dev2 = copy.copy(dev)
            dev2.stream, dev2.second = hip.hip_stream_create(dev), None
            self.more_work.append(self._work_set(dev2, ((self.chunk + 1) // 2 + 127) // 128 * 128))      # (a part: up to half a chunk, rounded up to whole tiles of 128 tokens)
        while len(self._keys_ev) < k:
            self._keys_ev.append([hip.hip_event_create(dev) for _ in self.layers])
            self._join_ev.append(hip.hip_event_create(dev))
        works = [self.work] + self.more_work[:k - 1]
        hip.hip_event_record(self._join_ev[0], dev.stream)            # the other streams after what this one holds so far
        for w in works[1:]:
            hip.hip_stream_wait(w.dev.stream, self._join_ev[0])
        gens = [self._steps(tokens[j * per:(j + 1) * per], self.pos + j * per, logits and j == k - 1, works[j]) for j in range(k)]
        for li in range(len(self.layers)):
            for j in range(k):
                assert next(gens[j]) == ("keys", li)
                if j < k - 1:
                    hip.hip_event_record(self._keys_ev[j][li], works[j].dev.stream)
                for i in range(j):
                    hip.hip_stream_wait(works[j].dev.stream, self._keys_ev[i][li])
            for j in range(k):
                assert next(gens[j]) == ("layer", li)
        for g in gens:
            for _ in g:
                pass
        for j in range(1, k):
            hip.hip_event_record(self._join_ev[j], works[j].dev.stream)
            hip.hip_stream_wait(dev.stream, self._join_ev[j])
        self.pos += n
        return self.logits

    def eval_tokens(self, tokens, logits=True):
        """The prompt in chunks (CUDA-EVAL, cuda-dense.lisp:295-305); the logits of the last token only.  A chunk of
        PARTS_FROM to PARTS_UPTO tokens goes as two or four parts side by side where that was measured to gain
        (forward_parts)."""
        tokens = list(tokens)
        for i in range(0, len(tokens), self.chunk):
            part = tokens[i:i + self.chunk]
            want = logits and i + len(part) >= len(tokens)
            npart = len(part)
            # Parts, measured on the Qwen3-4B shape (whole -> parts): 256 tokens 14.6 -> 14.0 ms, 512 18.7 -> 17.9 as halves;
            # 900 31.7 -> 28.0, 1,024 33.0 -> 30.2, 1,100 37.6 -> 33.8, 1,280 42.9 -> 40.8, 1,536 53.3 -> 50.4, 1,800 68.2 -> 64.0 as
            # halves (thirds and quarters of those lose); 2,048 78.8 -> 76.7 as halves, 72.1 as quarters.  Between 256 and 900
            # tokens only the powers of two gain (384 +8 %, but 448 -2 %, 640 0, 768 -1 to -6 %).  A chunk of 512 tokens far
            # into a long prompt is mostly attention, and its halves gain nothing (4,096 tokens in chunks of 512: 256.5 ->
            # 258-266 ms).  The bf16 products from the quantized matrices: two halves from 1,024 tokens on (1,024 tokens
            # 29.5 -> 26.1 ms, 2,048 66.7 -> 62.7; quarters lose, and so do halves of a 512-token chunk; their sums' order
            # depends on a launch's token count with or without parts); from resident copies 28.4 -> 27.2 and 62.7 -> 62.1:
            # left whole.  And a small model's launches are over before the next is queued, so twice as many of them only
            # cost (the Qwen2.5-0.5B shape's 512-token prompt 7.7 -> 10.6 ms as halves): a part must bring PARTS_WORK products
            # of a weight and a token to a layer (the Qwen3-4B shape's halves of 128 tokens bring 1.3e10, the 0.5B shape's
            # halves of 256 tokens 3.8e9).
            exact = self.prefill == "exact"
            k = 4 if exact and npart >= 2048 else 2
            c = self.c
            layer_weights = c["d"] * (2 * self.qd + 2 * self.kvd + 3 * c["ffn"])
            fits = npart >= 896 or (npart & (npart - 1) == 0 and self.pos < 1024)
            if ((exact and fits) or (self.prefill == "bf16" and npart >= 1024)) and PARTS_FROM <= npart <= PARTS_UPTO \
                    and (npart // k) * layer_weights >= PARTS_WORK:
                self.forward_parts(part, logits=want, k=k)
            else:
                self.forward_n(part, logits=want)

    def argmax(self):
        """The greedy token of self.logits (ARGMAX, model.lisp:464-468: the first of equal ones)."""
        return int(np.argmax(hip.hip_floats(self.logits, self.c["vocab"])))

    def free(self):
        for L in self.layers:
            for v in L.values():
                (v.free if hasattr(v, "free") else lambda: hip.hip_free(v))()
        if self.output is not self.embd:
            self.output.free()
        self.embd.free()
        for b in (self.output_norm, self.rope, self.logits):
            hip.hip_free(b)
        self._free_work(self.work)
        for w in self.more_work:                      # (hip_free waits for the device: nothing is in flight on these streams)
            self._free_work(w)
            if getattr(w.dev, "second", None) is not None:
                hip.hip_stream_destroy(w.dev.second)
                hip.hip_event_destroy(w.dev.forked)
                hip.hip_event_destroy(w.dev.joined)
            hip.hip_stream_destroy(w.dev.stream)
        for e in [e for evs in self._keys_ev for e in evs] + self._join_ev:
            hip.hip_event_destroy(e)
        self.more_work, self._keys_ev, self._join_ev = [], [], []
        for b in self.wb.values():
            hip.hip_free(b)
