"""The routed and shared experts of one FFN on the device: the host side of the
reference's DK-FFN-TAIL (src/cuda-ds4f.lisp:908-956, one token) and DK-FFN-ROUTED-CHUNK
(src/cuda-ds4f-prefill.lisp:315-356, a chunk), driving the kernels through LAUNCH.

An expert slot holds gate | up | down contiguously (cuda-ds4f.lisp:162-166): kernels get a
table of slot addresses and a byte offset (0, gate-bytes, 2 gate-bytes).  With 288 GB of
HBM every expert is resident, so there is no pool, no read-through and no CPU expert: slot
e is expert e.

Activations are quantized as the reference's CPU path quantizes them (Q8_K for the routed
experts, D4-ROUTED!, ds4f.lisp:994-1037; Q8_0 with a float scale for the shared expert,
D4-SHARED!, :1039-1048), not left as floats as its CUDA kernels take them.
"""
import ctypes as C

import numpy as np

from . import dense, hip
from .synth import IQ2_XXS, Q2_K, Q8_0, row_bytes


class ExpertPool:
    """NE experts on DEV, slot e = gate | up | down of expert e, 256-byte aligned.  The experts in HOST_EXPERTS stay
    in pinned host memory instead and are read through from there by the same kernels, their table entries pointing
    at it (what the reference's srcs[z] gives an expert without a slot, ds4f.cu:742-760): for a pool larger than the
    device's memory; with 288 GB every expert of a layer set fits and the default keeps all of them in HBM."""

    def __init__(self, dev, ne, d, ff, gate, up, down, host_experts=()):
        self.dev, self.ne, self.d, self.ff = dev, ne, d, ff
        self.grb, self.drb = row_bytes(IQ2_XXS, d), row_bytes(Q2_K, ff)
        self.gate_bytes, self.down_bytes = ff * self.grb, d * self.drb
        self.slot_bytes = (2 * self.gate_bytes + self.down_bytes + 255) // 256 * 256
        host = np.zeros((ne, self.slot_bytes), np.uint8)
        host[:, :self.gate_bytes] = np.asarray(gate, np.uint8).reshape(ne, self.gate_bytes)
        host[:, self.gate_bytes:2 * self.gate_bytes] = np.asarray(up, np.uint8).reshape(ne, self.gate_bytes)
        host[:, 2 * self.gate_bytes:2 * self.gate_bytes + self.down_bytes] = np.asarray(down, np.uint8).reshape(ne, self.down_bytes)
        self.pool = hip.hip_upload_new(dev, host)
        self.host_experts = sorted(set(int(e) for e in host_experts))
        self.host_buf = 0
        if self.host_experts:
            import ctypes
            self.host_buf = hip.hip_host_alloc(dev, len(self.host_experts) * self.slot_bytes)
            for i, e in enumerate(self.host_experts):
                ctypes.memmove(self.host_buf + i * self.slot_bytes, host[e].ctypes.data, self.slot_bytes)
                hip.hip_zero(hip.DBuf(self.slot_ptr_device(e), self.slot_bytes, dev))      # the device slot plays no part
        self.ptrs = hip.hip_upload_new(dev, np.array([self.slot_ptr(e) for e in range(ne)], np.uint64))

    def slot_ptr_device(self, e):
        return self.pool.ptr + int(e) * self.slot_bytes

    def slot_ptr(self, e):
        if int(e) in self.host_experts:
            return self.host_buf + self.host_experts.index(int(e)) * self.slot_bytes
        return self.slot_ptr_device(e)

    def free(self):
        hip.hip_sync(self.dev)
        hip.hip_free(self.pool)
        hip.hip_free(self.ptrs)
        if self.host_buf:
            hip.hip_host_free(self.host_buf)
            self.host_buf = 0


class SharedExpert:
    """The shared expert's three Q8_0 matrices, repacked (d4-upload-weights)."""

    def __init__(self, dev, d, ff, sgate, sup, sdown):
        from .dense import upload_gmat
        self.d, self.ff = d, ff
        self.gate = upload_gmat(dev, "ffn_gate_shexp", Q8_0, ff, d, sgate)
        self.up = upload_gmat(dev, "ffn_up_shexp", Q8_0, ff, d, sup)
        self.down = upload_gmat(dev, "ffn_down_shexp", Q8_0, d, ff, sdown)
        self.ones = None

    def free(self):
        for m in (self.gate, self.up, self.down):
            m.free()
        hip.hip_free(self.ones)


def _q8k(dev, x, n_elems, alloc=hip.hip_alloc):
    kq, kd = alloc(dev, n_elems), alloc(dev, 4 * n_elems // 256)
    ks = alloc(dev, 4 * n_elems // 16)
    hip.launch(dev, "quant_q8k", n_elems // 256, 256, [x, kq, kd, ks, hip.I64(n_elems // 256)])
    return kq, kd, ks


def ffn_shared(dev, sh, norm2, clamp, n=1, ws=None):
    """The shared expert of N tokens' NORM2 (DK-FFN-HEAD's second half): returns SOUT.
    With a Workspace WS nothing is allocated, freed or waited for."""
    d, ff = sh.d, sh.ff
    A = ws.alloc if ws else hip.hip_alloc
    qn_q, qn_s = A(dev, n * d), A(dev, 4 * n * d // 32)
    sg, su, smid = (A(dev, 4 * n * ff) for _ in range(3))
    qm_q, qm_s = A(dev, n * ff), A(dev, 4 * n * ff // 32)
    sout = A(dev, 4 * n * d)
    if getattr(sh, "ones", None) is None or sh.ones.bytes < 4 * n:
        sh.ones = hip.hip_upload_new(dev, np.ones(n, np.float32))
    one = sh.ones
    hip.launch(dev, "d4_quant", (n * d + 255) // 256, 256, [norm2, qn_q, qn_s, n * d // 32])
    if n == 1:
        hip.launch(dev, "d4_mvq8", (ff + 3) // 4, 128, [ff, d, ff, sh.gate.qs, sh.gate.d, qn_q, qn_s, sg])
        hip.launch(dev, "d4_mvq8", (ff + 3) // 4, 128, [ff, d, ff, sh.up.qs, sh.up.d, qn_q, qn_s, su])
    else:
        for w, y in ((sh.gate, sg), (sh.up, su)):
            hip.launch(dev, "mm_q8", ((n + 63) // 64, (ff + 63) // 64), 256, [w.qs, w.d, qn_q, qn_s, y, None, ff, d, n, 0])
    hip.launch(dev, "d4_swiglu_w", (n * ff + 255) // 256, 256, [n, ff, float(clamp), sg, su, one, smid, qm_q, qm_s])
    if n == 1:
        hip.launch(dev, "d4_mvq8", (d + 3) // 4, 128, [d, ff, d, sh.down.qs, sh.down.d, qm_q, qm_s, sout])
    else:
        hip.launch(dev, "mm_q8", ((n + 63) // 64, (d + 63) // 64), 256, [sh.down.qs, sh.down.d, qm_q, qm_s, sout, None, d, ff, n, 0])
    if ws:
        return sout
    hip.hip_sync(dev)
    for b in (qn_q, qn_s, sg, su, smid, qm_q, qm_s):
        hip.hip_free(b)
    return sout


def dk_mm(dev, kernel, w, wd, rbytes, rows, cols, x, y, n, x_stride=None, y_stride=None):
    """Y (N rows, Y-STRIDE apart) = W X (N rows, X-STRIDE apart): D4_MM_<format> (DK-MM, cuda-ds4f-prefill.lisp:65-68)."""
    hip.launch(dev, kernel, ((n + 63) // 64, (rows + 63) // 64), 128,
               [cols, rows, n, rbytes, cols if x_stride is None else x_stride, rows if y_stride is None else y_stride, w, wd, x, y])


def ffn_shared_chunk(dev, sh, norm2, n, clamp, ws=None):
    """The shared expert of a chunk of N tokens (DK-FFN-HEAD-CHUNK's second half, cuda-ds4f-prefill.lisp:294-298):
    gate and up through D4_MM_Q8_0 on the float rows, the gated activation, down through D4_MM_Q8_0.  Each token's
    row has d4-shared!'s bits.  Returns SOUT (N x d)."""
    d, ff = sh.d, sh.ff
    A = ws.alloc if ws else hip.hip_alloc
    sg, su, smid, sout = A(dev, 4 * n * ff), A(dev, 4 * n * ff), A(dev, 4 * n * ff), A(dev, 4 * n * d)
    if getattr(sh, "ones", None) is None or sh.ones.bytes < 4 * n:
        sh.ones = hip.hip_upload_new(dev, np.ones(n, np.float32))
    dk_mm(dev, "d4_mm_q8_0", sh.gate.qs, sh.gate.d, 0, ff, d, norm2, sg, n)
    dk_mm(dev, "d4_mm_q8_0", sh.up.qs, sh.up.d, 0, ff, d, norm2, su, n)
    hip.launch(dev, "d4_swiglu_w", (n * ff + 255) // 256, 256, [n, ff, float(clamp), sg, su, sh.ones, smid, None, None])
    dk_mm(dev, "d4_mm_q8_0", sh.down.qs, sh.down.d, 0, d, ff, smid, sout, n)
    if ws:
        return sout
    hip.hip_sync(dev)
    for b in (sg, su, smid):
        hip.hip_free(b)
    return sout


def tail_tables(dev, pool, sel, w):
    """The device tables DK-FFN-TAIL's kernels take for one token: the 2k matrix addresses
    (the selected experts' gates, then their ups) and the k weights."""
    gb = pool.gate_bytes
    ptrs = hip.hip_upload_new(dev, np.array([pool.slot_ptr(e) for e in sel] + [pool.slot_ptr(e) + gb for e in sel], np.uint64))
    return ptrs, hip.hip_upload_new(dev, np.asarray(w, np.float32))


def ffn_tail(dev, pool, sel, w, norm2, sout, clamp, keep=None, ws=None, tables=None):
    """One token's routed experts SEL (weights W) on NORM2, summed in SEL's order with the
    shared expert's SOUT (DK-FFN-TAIL, cuda-ds4f.lisp:908-956, its launches with its argument lists):
    gate and up in one launch over 2k matrices, the gated activation, down, the ordered sum; the
    expert kernels quantize their float rows themselves (Q8_K, as the CPU path does).  Returns MOE.
    With a Workspace WS nothing is allocated, freed or waited for; TABLES = tail_tables()
    made beforehand."""
    d, ff, k = pool.d, pool.ff, len(sel)
    gb = pool.gate_bytes
    A = ws.alloc if ws else hip.hip_alloc
    ptrs, bw = tables if tables else tail_tables(dev, pool, sel, w)
    bgu, bm = A(dev, 4 * 2 * k * ff), A(dev, 4 * k * ff)
    bd, moe = A(dev, 4 * k * d), A(dev, 4 * d)
    hip.launch(dev, "d4_mv_iq2_xxs", ((ff + 7) // 8, 1, 2 * k), 64,
               [d, ff, pool.grb, hip.I64(0), 0, ff, ptrs, None, norm2, bgu, None, None])
    hip.launch(dev, "d4_swiglu_w", (k * ff + 255) // 256, 256, [k, ff, float(clamp), bgu, bgu.at(4 * k * ff), bw, bm, None, None])
    hip.launch(dev, "d4_mv_q2_k", ((d + 7) // 8, 1, k), 64,
               [ff, d, pool.drb, hip.I64(2 * gb), ff, d, ptrs, None, bm, bd, None, None])
    hip.launch(dev, "d4_moe_sum", (d + 255) // 256, 256, [d, k, bd, sout, moe, None])
    if ws:
        return moe
    hip.hip_sync(dev)
    if keep is not None:
        keep["mid"] = hip.hip_floats(bm, k * ff).reshape(k, ff)
        keep["gu"] = hip.hip_floats(bgu, 2 * k * ff).reshape(2, k, ff)
        keep["down"] = hip.hip_floats(bd, k * d).reshape(k, d)
    for b in (bgu, bm, bd) + (() if tables else (ptrs, bw)):
        hip.hip_free(b)
    return moe


def fused_tables(dev, pool, sel, w):
    """The device tables the fused decode step takes for one token: the k slot addresses and
    the k weights."""
    return (hip.hip_upload_new(dev, np.array([pool.slot_ptr(e) for e in sel], np.uint64)),
            hip.hip_upload_new(dev, np.asarray(w, np.float32)))


def ffn_step_fused(dev, pool, sh, sel, w, norm2, clamp, ws=None, tables=None, routed=None):
    """One token's shared expert and routed experts in five launches, with ffn_shared's and
    ffn_tail's bits: the shared expert's gate, up and gated activation in one launch and its
    down in one (both quantizing their float input in the kernel); the routed experts' gates,
    ups and gated activations in one launch over k expert slots, their downs in one, then
    the ordered sum.  Returns MOE.  ROUTED = (sel, w) DBufs as d4_route left them on the
    device (k of them): the kernels then index the pool's slot table by sel themselves and
    SEL, W are not used (pass k as SEL)."""
    d, ff = pool.d, pool.ff
    k = sel if routed else len(sel)
    gb = pool.gate_bytes
    A = ws.alloc if ws else hip.hip_alloc
    dsel = None
    if routed:
        ptrs, (dsel, bw), tables = pool.ptrs, routed, True
    else:
        ptrs, bw = tables if tables else fused_tables(dev, pool, sel, w)
    smid, sout = A(dev, 4 * ff), A(dev, 4 * d)
    bm, bd, moe = A(dev, 4 * k * ff), A(dev, 4 * k * d), A(dev, 4 * d)
    hip.launch(dev, "d4_mvq8_glu", (ff + 3) // 4, 128, [ff, d, sh.gate.qs, sh.gate.d, sh.up.qs, sh.up.d, norm2, float(clamp), smid])
    dense.mv_multi(dev, [(sh.down, sout, None)], xf=smid, f16_scale=False)
    hip.launch(dev, "d4_mv_glu_iq2_xxs", ((ff + 7) // 8, 1, k), 64,
               [d, ff, pool.grb, hip.I64(0), hip.I64(gb), 0, ff, ptrs, dsel, norm2, bw, float(clamp), bm])
    hip.launch(dev, "d4_mv_q2_k_f32", ((d + 7) // 8, 1, k), 64, [ff, d, pool.drb, hip.I64(2 * gb), ff, d, ptrs, dsel, bm, bd])
    hip.launch(dev, "d4_moe_sum", (d + 255) // 256, 256, [d, k, bd, sout, moe, None])
    if ws:
        return moe
    hip.hip_sync(dev)
    for b in (smid, sout, bm, bd) + (() if tables else (ptrs, bw)):
        hip.hip_free(b)
    return moe


def ffn_step_device(dev, pool, sh, logits, norm2, ne, nu, scale, clamp, bias=None, ws=None, tid2eid=None, tokens=None):
    """A decode step with nothing going through the host: d4_route on the device, then
    ffn_step_fused indexing the slot table by its result (six launches).  TID2EID, TOKENS:
    a hash layer's table and the token's id on the device (see route)."""
    A = ws.alloc if ws else hip.hip_alloc
    sel, w = route(dev, logits, 1, ne, nu, scale, bias, A, tid2eid=tid2eid, tokens=tokens)
    moe = ffn_step_fused(dev, pool, sh, nu, None, norm2, clamp, ws=ws, routed=(sel, w))
    if not ws:
        hip.hip_free(sel); hip.hip_free(w)
    return moe


class FfnStepWeights(C.Structure):
    """ilt_ffn_step_weights: the slot table and the shared expert's repacked matrices."""
    _fields_ = [("slots", C.c_uint64), ("gate_bytes", C.c_int64),
                ("sgate_q", C.c_uint64), ("sgate_d", C.c_uint64), ("sup_q", C.c_uint64), ("sup_d", C.c_uint64),
                ("sdown_q", C.c_uint64), ("sdown_d", C.c_uint64)]


def step_weights(pool, sh):
    return FfnStepWeights(pool.ptrs.ptr, pool.gate_bytes, sh.gate.qs.ptr, sh.gate.d.ptr, sh.up.qs.ptr, sh.up.d.ptr,
                          sh.down.qs.ptr, sh.down.d.ptr)


def step_workspace_bytes(nu, d, ff):
    f = hip.lib().ilt_d4_ffn_step_workspace
    f.restype = C.c_uint64
    return int(f(C.c_int(nu), C.c_int(d), C.c_int(ff)))


def ffn_step_call(dev, pool, sh, logits, norm2, moe, ne, nu, scale, clamp, bias=None, wsbuf=None):
    """ffn_step_device's step queued by one call into the library (ilt_d4_ffn_step; four launches, the routing carried
    along by the shared expert's gate/up launch and the ordered sum by its down launch where those launches are the
    streamed ones, else one launch more for each): the
    host crosses the boundary once a layer instead of once a launch.  WSBUF: a DBuf of
    step_workspace_bytes for the intermediate results (one is made and freed if None);
    MOE: the output DBuf (d floats)."""
    own = wsbuf is None
    if own:
        wsbuf = hip.hip_alloc(dev, step_workspace_bytes(nu, pool.d, pool.ff), zero=False)
    wt = step_weights(pool, sh)
    hip.call("ilt_d4_ffn_step", C.c_uint64(dev.stream), C.c_uint64(wsbuf.ptr), C.c_uint64(wsbuf.bytes), C.c_int(ne), C.c_int(nu),
             C.c_int(pool.d), C.c_int(pool.ff), C.c_float(scale), C.c_float(clamp), C.byref(wt), C.c_uint64(logits.ptr),
             C.c_uint64(bias.ptr if bias is not None else 0), C.c_uint64(norm2.ptr), C.c_uint64(moe.ptr))
    if own:
        hip.hip_sync(dev)
        hip.hip_free(wsbuf)
    return moe


def ffn_step_noalloc(dev, pool, sh, logits, norm2, moe, ne, nu, scale, clamp, bias=None):
    """ffn_step_call with the intermediate results in the library's own device array
    (ilt_d4_ffn_step_noalloc): no workspace, no allocation; steps of more than 1 MiB of
    intermediates raise.  Calls that overlap on one GPU race on the array."""
    wt = step_weights(pool, sh)
    hip.call("ilt_d4_ffn_step_noalloc", C.c_uint64(dev.stream), C.c_int(ne), C.c_int(nu), C.c_int(pool.d), C.c_int(pool.ff),
             C.c_float(scale), C.c_float(clamp), C.byref(wt), C.c_uint64(logits.ptr),
             C.c_uint64(bias.ptr if bias is not None else 0), C.c_uint64(norm2.ptr), C.c_uint64(moe.ptr))
    return moe


def ffn_small(dev, pool, sh, logits, norm2, n, ne, nu, scale, clamp, bias=None, grouped=False):
    """The FFN past the router for a short pass's N <= 9 tokens (DK-FFN-SMALL,
    cuda-ds4f-spec.lisp:30-100: a speculative step's verification), every token with decode's
    bits.  The reference routes on the CPU and hands each expert its tokens' rows through
    counts/bases; here d4_route leaves sel and the weights on the device and the expert
    kernels take one slot per (token, slot) row, row t*nu + j on expert sel[t*nu + j]: the
    gathered rows, gate+up+gated activation of all rows in one launch, their downs in one, the
    sums in slot order with the shared expert's (d4_mvq8n for its three products).  Returns
    MOE (N x d).  GROUPED "counts": DK-FFN-SMALL's own launches with its argument lists
    (cuda-ds4f-spec.lisp:82-88) -- d4_gather_rows, d4_mv_iq2_xxs for the gates and again for the ups,
    d4_swiglu_w, d4_mv_q2_k, each expert kernel over all NE slots with the counts and bases that
    d4_group_* left on the device (an expert nobody chose has a count of 0)."""
    d, ff = pool.d, pool.ff
    rows = n * nu
    gb = pool.gate_bytes
    A = hip.hip_alloc
    # the shared expert on the N tokens
    qn_q, qn_s = A(dev, n * d), A(dev, 4 * n * d // 32)
    sg, su, smid = (A(dev, 4 * n * ff) for _ in range(3))
    qm_q, qm_s = A(dev, n * ff), A(dev, 4 * n * ff // 32)
    sout = A(dev, 4 * n * d)
    one = hip.hip_upload_new(dev, np.ones(n, np.float32))
    hip.launch(dev, "d4_quant", (n * d + 255) // 256, 256, [norm2, qn_q, qn_s, n * d // 32])
    hip.launch(dev, "d4_mvq8n", (ff + 3) // 4, 128, [ff, d, ff, n, d, ff, sh.gate.qs, sh.gate.d, qn_q, qn_s, sg])
    hip.launch(dev, "d4_mvq8n", (ff + 3) // 4, 128, [ff, d, ff, n, d, ff, sh.up.qs, sh.up.d, qn_q, qn_s, su])
    hip.launch(dev, "d4_swiglu_w", (n * ff + 255) // 256, 256, [n, ff, float(clamp), sg, su, one, smid, qm_q, qm_s])
    hip.launch(dev, "d4_mvq8n", (d + 3) // 4, 128, [d, ff, d, n, ff, d, sh.down.qs, sh.down.d, qm_q, qm_s, sout])
    # the routed experts: row r = (token r / nu, slot r % nu)
    sel, w = route(dev, logits, n, ne, nu, scale, bias)
    extra = []
    if grouped == "counts":
        g = group_rows(dev, sel, w, n, ne, nu)
        rmap, smap, wrow = g["rmap"], g["smap"], g["wrow"]
        x, bg, bu = A(dev, 4 * rows * d), A(dev, 4 * rows * ff), A(dev, 4 * rows * ff)
        bm, bd, moe = A(dev, 4 * rows * ff), A(dev, 4 * rows * d), A(dev, 4 * n * d)
        hip.launch(dev, "d4_gather_rows", (rows * d + 255) // 256, 256, [d, rows, norm2, rmap, x])
        for add, out in ((0, bg), (gb, bu)):
            hip.launch(dev, "d4_mv_iq2_xxs", ((ff + 7) // 8, 1, ne), 64,
                       [d, ff, pool.grb, hip.I64(add), d, ff, pool.ptrs, None, x, out, g["counts"], g["bases"]])
        hip.launch(dev, "d4_swiglu_w", (rows * ff + 255) // 256, 256, [rows, ff, float(clamp), bg, bu, wrow, bm, None, None])
        hip.launch(dev, "d4_mv_q2_k", ((d + 7) // 8, 1, ne), 64,
                   [ff, d, pool.drb, hip.I64(2 * gb), ff, d, pool.ptrs, None, bm, bd, g["counts"], g["bases"]])
        hip.launch(dev, "d4_moe_sum_rows", (n * d + 255) // 256, 256, [d, nu, n, bd, smap, sout, moe])
        hip.hip_sync(dev)
        for b in [qn_q, qn_s, sg, su, smid, qm_q, qm_s, sout, one, sel, w, x, bg, bu, bm, bd] + list(g.values()):
            hip.hip_free(b)
        return moe
    if grouped:
        # GROUPED: the rows grouped by expert on the device (d4_group_*), an expert's rows one after another, so its
        # matrices come from memory once for all its tokens: what the reference's counts / bases arguments give
        g = group_rows(dev, sel, w, n, ne, nu)
        rmap, smap, wrow = g["rmap"], g["smap"], g["wrow"]
        rexp = A(dev, 4 * rows)
        hip.launch(dev, "d4_rows_expert", (rows + 255) // 256, 256, [rows, sel, smap, rexp])
        extra = [rexp] + [v for k, v in g.items() if k not in ("rmap", "smap")]
    else:
        rmap = hip.hip_upload_new(dev, (np.arange(rows) // nu).astype(np.uint32))
        smap = hip.hip_upload_new(dev, np.arange(rows, dtype=np.uint32))
        rexp, wrow = sel, w
    x, bm, bd, moe = A(dev, 4 * rows * d), A(dev, 4 * rows * ff), A(dev, 4 * rows * d), A(dev, 4 * n * d)
    hip.launch(dev, "d4_gather_rows", (rows * d + 255) // 256, 256, [d, rows, norm2, rmap, x])
    hip.launch(dev, "d4_mv_glu_iq2_xxs", ((ff + 7) // 8, 1, rows), 64,
               [d, ff, pool.grb, hip.I64(0), hip.I64(gb), d, ff, pool.ptrs, rexp, x, wrow, float(clamp), bm])
    hip.launch(dev, "d4_mv_q2_k_f32", ((d + 7) // 8, 1, rows), 64, [ff, d, pool.drb, hip.I64(2 * gb), ff, d, pool.ptrs, rexp, bm, bd])
    hip.launch(dev, "d4_moe_sum_rows", (n * d + 255) // 256, 256, [d, nu, n, bd, smap, sout, moe])
    hip.hip_sync(dev)
    for b in [qn_q, qn_s, sg, su, smid, qm_q, qm_s, sout, one, sel, w, rmap, smap, x, bm, bd] + extra:
        hip.hip_free(b)
    return moe


def route(dev, logits, n, ne, nu, scale, bias=None, alloc=hip.hip_alloc, tid2eid=None, tokens=None):
    """D4_ROUTE for N tokens' LOGITS (a DBuf): returns (sel, w) DBufs of N x NU.  On a hash layer
    (d4-route, ds4f.lisp:961-963; DK-FFN-ROUTED-CHUNK passes HASH 1, cuda-ds4f-prefill.lisp) TID2EID is
    the layer's table on the device (int32, NU experts a vocabulary entry) and TOKENS the N token ids
    (uint32): token t's experts are its row of the table as it stands, the weights from the logits."""
    if (tid2eid is None) != (tokens is None):
        raise ValueError("a hash layer's routing takes both the table and the token ids")
    sel, w = alloc(dev, 4 * n * nu), alloc(dev, 4 * n * nu)
    hip.launch(dev, "d4_route", n, ne, [ne, nu, 0 if tid2eid is None else 1, float(scale), 1 if bias is not None else 0, logits, bias,
                                        tid2eid, tokens, sel, w],
               shared=4 * (2 * ne + 64 + nu))
    return sel, w


def group_rows(dev, sel, w, n, ne, nu, alloc=hip.hip_alloc):
    """The N x NU (token, slot) rows grouped by expert (D4_GROUP_*): returns a dict of DBufs
    counts, bases (per expert), rmap (row -> token), smap ((token, slot) -> row), wrow."""
    rows = n * nu
    g = {k: alloc(dev, 4 * (ne if k in ("counts", "bases") else rows)) for k in
         ("counts", "bases", "rank", "rmap", "smap", "wrow")}
    hip.launch(dev, "d4_group_zero", (ne + 255) // 256, min(ne, 256), [ne, g["counts"]])
    hip.launch(dev, "d4_group_count", (rows + 255) // 256, 256, [rows, ne, nu, sel, g["counts"], g["rank"]])
    hip.launch(dev, "d4_group_scan", 1, ne, [rows, ne, nu, g["counts"], g["bases"]])
    hip.launch(dev, "d4_group_scatter", (rows + 255) // 256, 256,
               [rows, ne, nu, sel, g["rank"], g["bases"], w, g["rmap"], g["smap"], g["wrow"]])
    return g


def ffn_routed_chunk_bf16(dev, pool, logits, norm2, sout, n, ne, nu, scale, clamp, bias=None, keep=None, ws=None, fused=None):
    """FFN-ROUTED-CHUNK with the three grouped products on the bf16 matrix cores: the same
    routing, grouping, gated activation and slot-ordered sum, no activation quantizers and no
    gathered copy (the gate and up products read the tokens' rows through the row map).
    Within 2e-2 of the CPU path's chunk; the routing and grouping stay exact.  With a
    Workspace WS nothing is allocated, freed or waited for.  FUSED: gate, up and the gated
    activation in one launch (the same bits; needs ff a multiple of 128); None = whenever
    nobody asks to KEEP the two products."""
    d, ff = pool.d, pool.ff
    if fused is None:
        fused = keep is None and ff % 128 == 0
    rows = n * nu
    gb = pool.gate_bytes
    A = ws.alloc if ws else hip.hip_alloc
    sel, w = route(dev, logits, n, ne, nu, scale, bias, A)
    g = group_rows(dev, sel, w, n, ne, nu, A)
    ptrs = pool.ptrs
    xb = dense.cvt_bf16(dev, norm2, n * d, A(dev, 2 * n * d))
    gg, gu = (A(dev, 4 * rows * ff) for _ in range(2)) if not fused else (None, None)
    mb = A(dev, 2 * rows * ff)
    down, moe = A(dev, 4 * rows * d), A(dev, 4 * n * d)

    def mm_id(qtype, ncols, nrows, rb, add, xin, rmap, yout):
        hip.launch(dev, "d4_mm_id_bf16", (rows // 128 + ne, (nrows + 127) // 128), 256,
                   [qtype, ncols, nrows, rb, hip.I64(add), ptrs, g["counts"], g["bases"], ne, hip.I64(rows), xin, rmap, yout])

    if fused:
        hip.launch(dev, "d4_mm_id_glu_bf16", (rows // 128 + ne, ff // 128), 256,
                   [IQ2_XXS, d, ff, pool.grb, hip.I64(0), hip.I64(gb), ptrs, g["counts"], g["bases"], ne, hip.I64(rows), xb, g["rmap"],
                    float(clamp), g["wrow"], mb])
    else:
        mm_id(IQ2_XXS, d, ff, pool.grb, 0, xb, g["rmap"], gg)
        mm_id(IQ2_XXS, d, ff, pool.grb, gb, xb, g["rmap"], gu)
        hip.launch(dev, "d4_swiglu_w_bf16", (rows * ff // 8 + 255) // 256, 256, [rows, ff, float(clamp), gg, gu, g["wrow"], mb])
    mm_id(Q2_K, ff, d, pool.drb, 2 * gb, mb, None, down)
    hip.launch(dev, "d4_moe_sum_rows", (n * d + 255) // 256, 256, [d, nu, n, down, g["smap"], sout, moe])
    if ws:
        return moe
    hip.hip_sync(dev)
    if keep is not None:
        keep["sel"] = hip.hip_download(sel, np.uint32, rows).reshape(n, nu)
        keep["w"] = hip.hip_floats(w, rows).reshape(n, nu)
        keep["counts"] = hip.hip_download(g["counts"], np.uint32, ne)
        keep["bases"] = hip.hip_download(g["bases"], np.uint32, ne)
        keep["rmap"] = hip.hip_download(g["rmap"], np.uint32, rows)
        keep["mid"] = (hip.hip_download(mb, np.uint16, rows * ff).astype(np.uint32) << 16).view(np.float32).reshape(rows, ff)
        if not fused:
            keep["gate"], keep["up"] = (hip.hip_floats(b, rows * ff).reshape(rows, ff) for b in (gg, gu))
        keep["down"] = hip.hip_floats(down, rows * d).reshape(rows, d)
    for b in [sel, w, xb, mb, down] + ([] if fused else [gg, gu]) + list(g.values()):
        hip.hip_free(b)
    return moe


def ffn_routed_chunk(dev, pool, logits, norm2, sout, n, ne, nu, scale, clamp, bias=None, keep=None, ws=None):
    """A chunk of N tokens past the router (DK-FFN-ROUTED-CHUNK): each token's experts and
    weights (d4_route), the (token, slot) rows grouped by expert, the rows gathered and
    quantized, every expert's gate, up and down as one grouped product each over its rows
    (d4_mm_id_*), the gated activation between, then each token's rows summed in slot order
    with the shared expert's SOUT.  LOGITS (N x NE), NORM2 (N x D) and SOUT (N x D) are
    DBufs; returns MOE (N x D).  With a Workspace WS nothing is allocated, freed or waited for."""
    d, ff = pool.d, pool.ff
    rows = n * nu
    gb = pool.gate_bytes
    A = ws.alloc if ws else hip.hip_alloc
    sel, w = route(dev, logits, n, ne, nu, scale, bias, A)
    g = group_rows(dev, sel, w, n, ne, nu, A)
    ptrs = pool.ptrs
    x = A(dev, 4 * rows * d)
    hip.launch(dev, "d4_gather_rows", (rows * d + 255) // 256, 256, [d, rows, norm2, g["rmap"], x])
    xq, xd, xs = _q8k(dev, x, rows * d, A)
    gg, gu, mid = (A(dev, 4 * rows * ff) for _ in range(3))
    down, moe = A(dev, 4 * rows * d), A(dev, 4 * n * d)

    def mm_id(kernel, ncols, nrows, rb, add, xin, yout):
        hip.launch(dev, kernel, ((n + 63) // 64, (nrows + 63) // 64, ne), 128,
                   [ncols, nrows, rb, ncols, nrows, hip.I64(add), ptrs, g["counts"], g["bases"], xin[0], yout,
                    xin[1], xin[2], hip.I64(rows)])

    mm_id("d4_mm_id_iq2_xxs", d, ff, pool.grb, 0, (xq, xd, None), gg)
    mm_id("d4_mm_id_iq2_xxs", d, ff, pool.grb, gb, (xq, xd, None), gu)
    hip.launch(dev, "d4_swiglu_w", (rows * ff + 255) // 256, 256, [rows, ff, float(clamp), gg, gu, g["wrow"], mid, None, None])
    mq, md, ms = _q8k(dev, mid, rows * ff, A)
    mm_id("d4_mm_id_q2_k", ff, d, pool.drb, 2 * gb, (mq, md, ms), down)
    hip.launch(dev, "d4_moe_sum_rows", (n * d + 255) // 256, 256, [d, nu, n, down, g["smap"], sout, moe])
    if ws:
        return moe
    hip.hip_sync(dev)
    if keep is not None:
        keep["sel"] = hip.hip_download(sel, np.uint32, rows).reshape(n, nu)
        keep["w"] = hip.hip_floats(w, rows).reshape(n, nu)
        keep["counts"] = hip.hip_download(g["counts"], np.uint32, ne)
    for b in [sel, w, x, xq, xd, xs, gg, gu, mid, mq, md, ms, down] + list(g.values()):
        hip.hip_free(b)
    return moe
