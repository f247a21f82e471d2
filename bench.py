#!/usr/bin/env python3
"""bench.py -- the quantized matrix-product path on one MI355X.

The default workload (c2) is the one the metric is quoted on: a step is one decoded token's
worth of quantized products at the Qwen3-4B shape (the benchmark's configuration 2) -- for each of
36 layers the activation quantizations (inside the product kernels) and the seven matrix-vector products (Q4_K wq
4096x2560, wk 1024x2560, wo 2560x4096, gate and up 9728x2560; Q6_K wv 1024x2560, down
2560x9728), then the Q6_K output head 151936x2560: 2,618,273,280 bytes of GGUF blocks
streamed from HBM per step, every matrix its own allocation, so the working set (2.6 GB)
is far beyond the 256 MB MALL.  No attention, norm or RoPE runs in a step: those belong to
the dense-forward harness, not to this path.

Without --workload the line is c2's, and the other configurations run after it on the same clock
and are reported under "configs" (c2_decode, c1, c1_decode, c3 and c5 on the bf16 matrix cores and on the exact
int8 path, c4 with the routing on the device); c2_decode's figures are also the line's
decode_tok_per_s, decode_ms_per_token and prefill_tok_per_s.

Other workloads (--workload), each the benchmark configuration of the same number:
  c2d the whole dense decoder at config 2's shape (36 layers, head norms, RoPE, attention over an
      fp32 KV cache): a 512-token prompt through the prefill products, then 256 greedy tokens,
      each picked on the device and fed on from device memory (--host-argmax: every token's
      logits downloaded and the next token picked on the host)
  c1  Q8_0 decode GEMV 4864x896 and 896x4864, rotating over 64 copies (593 MB)
  c3  Q6_K prefill product 17408x5120 on T tokens (--tokens, default 4096): bf16 matrix
      cores (--path bf16, the float activations rounded to bf16 inside the step) or the
      bit-exact int8 path (--path int8, the Q8_K activation quantizer inside the step)
  c4  MoE decode step: 256 resident experts (IQ2_XXS gate/up, Q2_K down), top-6, the Q8_0
      shared expert, rotating over 3 layers' pools (5.4 GB); routing tables made beforehand;
      --mode fused (default): 5 launches a step; --mode single: the reference's 12;
      --mode device: routing on the device inside the step, one call into the library (4 launches, no host tables)
  c5  MoE prefill chunk: 4096 tokens, Zipf(1.1)-skewed top-6 routing, route -> group ->
      gather -> grouped gate, up -> gated activation -> grouped down -> ordered sum
Weights and activations are synthetic and seeded (illatio_amd/synth.py); inputs are resident
in HBM before the timed region.

Prints one JSON line: the metric, the roofline of the dominant kernel (timed with HIP events
on the launch stream in a second pass over the same sequence) and the CPU oracle timed on a
bounded sample of the same workload on this host's cores.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

# HBM bytes per launch of the product kernels, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE (KiB per dispatch), as
# profiles/hbm_traffic_per_launch.md lists them (its header says how its rows were measured): FETCH_SIZE reads 0.500 of
# what a plain streaming kernel of known size fetches (cvt_bf16: 83,886,080 bytes read, counter 40,971 KiB), WRITE_SIZE
# reads 1.000 (same kernel: 41,943,040 bytes written, counter 40,960 KiB); so bytes = (2 * FETCH_SIZE + WRITE_SIZE) * 1024.
# The counters sit between a die's L2 and the fabric: bytes that come from the memory-side cache count like bytes from HBM.
def _t(fetch_kib, write_kib):
    return int((2 * fetch_kib + write_kib) * 1024)


def load_traffic(path=os.path.join(ROOT, "profiles", "hbm_traffic_per_launch.md")):
    """{workload: {launch: bytes}} from the table's rows `| workload | launch | kernel | FETCH_SIZE KiB | WRITE_SIZE KiB |`
    (several kernels of one launch shape: their rows add up)."""
    t = {}
    try:
        for line in open(path):
            cells = [c.strip() for c in line.strip().strip("|").split("|")]
            if len(cells) < 5 or cells[0] in ("workload", "") or set(cells[0]) <= set("-: "):
                continue
            try:
                b = _t(float(cells[3]), float(cells[4]))
            except ValueError:
                continue
            w = t.setdefault(cells[0], {})
            w[cells[1]] = w.get(cells[1], 0) + b
    except OSError:
        pass
    return t


TRAFFIC = load_traffic()


def traffic_of(workload, per):
    """Measured HBM bytes per launch, averaged over the launches the roofline entry covers."""
    t = TRAFFIC.get(workload, {})
    n = sum(v[2] for k, v in per.items() if k in t)
    return int(sum(t[k] * v[2] for k, v in per.items() if k in t) / n) if n else None


HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "bf16-1pass": 2500.0, "bf16-2pass": 2500.0, "bf16-resident": 2500.0, "int8": 5000.0, "int8-2pass": 5000.0,
                    "int8-resident": 5000.0}

D, FFN, QD, KVD, VOCAB, LAYERS = 2560, 9728, 4096, 1024, 151936, 36


def host_cores():
    """Physical cores this process may run on (hyperthreads counted once), at most the 16 of a one-GPU box's share."""
    try:
        allowed = set(os.sched_getaffinity(0))
    except AttributeError:
        allowed = set(range(os.cpu_count() or 1))
    cores = set()
    try:
        cpu = phys = core = None
        for line in open("/proc/cpuinfo"):
            k, _, v = line.partition(":")
            k, v = k.strip(), v.strip()
            if k == "processor":
                cpu, phys, core = int(v), None, None
            elif k == "physical id":
                phys = v
            elif k == "core id":
                core = v
            if cpu is not None and phys is not None and core is not None:
                if cpu in allowed:
                    cores.add((phys, core))
                cpu = None
    except OSError:
        pass
    n = len(cores) if cores else len(allowed)
    return max(1, min(n, 16))


def one_thread_figure(work_fn, seconds=3.0):
    """WORK_FN(nthreads) -> units of work done; its rate on one thread over about SECONDS."""
    t1, done = time.perf_counter(), 0.0
    while time.perf_counter() - t1 < seconds:
        done += work_fn(1)
    return done / (time.perf_counter() - t1)


class Timer:
    """K steps timed between two syncs, wall clock and device events; then the same
    sequence once more with an event pair around every launch that names a kernel."""

    def __init__(self, dev):
        from illatio_amd import hip
        self.hip, self.dev, self.probes, self.probing = hip, dev, [], False

    def launch(self, label, work, fn):
        """Run FN (one kernel launch); WORK = its algorithmic bytes or flops."""
        hip = self.hip
        if self.probing:
            e0, e1 = hip.hip_event_create(self.dev, True), hip.hip_event_create(self.dev, True)
            hip.hip_event_record(e0, self.dev.stream)
            fn()
            hip.hip_event_record(e1, self.dev.stream)
            self.probes.append((label, work, e0, e1))
        else:
            fn()

    def run(self, step, steps, warmup, probe_steps=3, work_of=None):
        """WORK_OF(kernel name, launch arguments) -> algorithmic work: when given, the probing
        pass puts an event pair around every launch the host functions make, by kernel name."""
        hip, dev = self.hip, self.dev
        for i in range(warmup):
            step(i)
        hip.hip_sync(dev)
        ev = [hip.hip_event_create(dev, timing=True) for _ in range(2)]
        t0 = time.perf_counter()
        hip.hip_event_record(ev[0], dev.stream)
        for i in range(steps):
            step(warmup + i)
        hip.hip_event_record(ev[1], dev.stream)
        self.enqueue_ms = (time.perf_counter() - t0) * 1e3 / steps     # host time to queue a step's launches
        hip.hip_sync(dev)
        wall_ms = (time.perf_counter() - t0) * 1e3
        dev_ms = hip.hip_event_elapsed_ms(ev[0], ev[1])
        self.probing = True
        plain = hip.launch
        if work_of:
            def probed(d, kernel, grid, block, a, shared=0):
                self.launch(kernel, work_of(kernel, a), lambda: plain(d, kernel, grid, block, a, shared))
            hip.launch = probed
        try:
            step(warmup + steps)                       # once unrecorded: a launch path the timed steps did not take is cold
            hip.hip_sync(dev)
            for e in self.probes:
                hip.hip_event_destroy(e[2]); hip.hip_event_destroy(e[3])
            self.probes = []
            for i in range(max(1, min(steps, probe_steps))):
                step(warmup + steps + i)
            hip.hip_sync(dev)
        finally:
            hip.launch = plain
        self.probing = False
        times = {}
        for label, work, e0, e1 in self.probes:
            t = times.setdefault(label, [[], 0])
            t[0].append(hip.hip_event_elapsed_ms(e0, e1)); t[1] += work
            hip.hip_event_destroy(e0); hip.hip_event_destroy(e1)
        # a kernel's time: the median of its launches (the events of a launch now and then take in a stall that is
        # not the kernel's), times their number
        per = {label: [float(np.median(ts)) * len(ts), work, len(ts)] for label, (ts, work) in times.items()}
        return max(wall_ms, dev_ms) / steps, dev_ms / steps, per


def roofline_of(per, bound, peak, unit, kernel_names):
    """The dominant kernel's roofline entry from the per-label (ms, work, launches) sums."""
    dom = max(per, key=lambda k: per[k][0])
    ms, work, n = per[dom]
    scale = 1e9 if unit == "GB/s" else 1e12
    achieved = work / (ms * 1e-3) / scale
    return {"bound": bound, "achieved": round(achieved, 1), "peak": peak, "unit": unit, "frac": round(achieved / peak, 4),
            "traffic": None, "kernel": kernel_names.get(dom, dom), "launches": n, "avg_launch_us": round(ms / n * 1e3, 2),
            "avg_work_per_launch": work // n,
            "other_kernels": {kernel_names.get(k, k): {unit: round(v[1] / (v[0] * 1e-3) / scale, 1), "launches": v[2],
                                                       "avg_launch_us": round(v[0] / v[2] * 1e3, 2)}
                              for k, v in per.items() if k != dom and v[1]}}


# ---------------------------------------------------------------------------------------------
def workload_c2(args, dev):
    from illatio_amd import dense, hip, synth
    rng = synth.make_rng(42)
    nl = args.layers
    specs = [("wq", synth.Q4_K, QD, D, "x"), ("wk", synth.Q4_K, KVD, D, "x"), ("wv", synth.Q6_K, KVD, D, "x"),
             ("wo", synth.Q4_K, D, QD, "att"), ("gate", synth.Q4_K, FFN, D, "x"), ("up", synth.Q4_K, FFN, D, "x"),
             ("down", synth.Q6_K, D, FFN, "mid")]
    host = {name: synth.weights(qt, rows, cols, rng) for name, qt, rows, cols, _ in specs}
    layers = [{name: dense.upload_gmat(dev, f"blk.{li}.{name}", qt, rows, cols, host[name])
               for name, qt, rows, cols, _ in specs} for li in range(nl)]
    head_host = synth.weights(synth.Q6_K, VOCAB, D, rng)
    head = dense.upload_gmat(dev, "output", synth.Q6_K, VOCAB, D, head_host)
    wbytes = {name: synth.row_bytes(qt, cols) * rows for name, qt, rows, cols, _ in specs}
    step_bytes = nl * sum(wbytes.values()) + head_host.size

    xin = {"x": D, "att": QD, "mid": FFN}
    xbuf = {k: hip.hip_upload_new(dev, synth.activations(n, rng)) for k, n in xin.items()}
    acts = {k: dense.QAct(dev, 1, n, ("q8k",)) for k, n in xin.items()}
    ybuf = {name: hip.hip_alloc(dev, 4 * rows) for name, _, rows, _, _ in specs}
    logits = hip.hip_alloc(dev, 4 * VOCAB)
    tm = Timer(dev)
    fused, inq = args.mode != "single", args.mode in ("fused", "device")
    # --norm: the layer's two norms and the output norm as well (rmsnorm!, model.lisp:205-216): inside the
    # product launches when they quantize for themselves, else as rmsnorm_q8k launches in the quantizers' place
    nwb = hip.hip_upload_new(dev, (synth.activations(D, rng) * 0.2 + 1.0).astype(np.float32)) if args.norm else None
    norm = (nwb, 1e-6) if (args.norm and inq) else None

    def quantize_x():
        if args.norm:
            dense.rmsnorm_q8(dev, xbuf["x"], nwb, acts["x"], D, 1e-6)
        else:
            dense.quantize_act(dev, xbuf["x"], acts["x"])

    def step(_):
        for L in layers:
            if fused:
                xf = xbuf["x"] if inq else None
                if not inq:
                    quantize_x()
                tm.launch("qkv", wbytes["wq"] + wbytes["wk"] + wbytes["wv"] + D + 4 * (QD + 2 * KVD),
                          lambda: dense.qkv_mul(dev, L["wq"], L["wk"], L["wv"], acts["x"], ybuf["wq"], ybuf["wk"], ybuf["wv"], xf=xf, norm=norm))
                if not inq:
                    dense.quantize_act(dev, xbuf["att"], acts["att"])
                tm.launch("wo", wbytes["wo"] + QD + 4 * D,
                          lambda: dense.mv_multi(dev, [(L["wo"], ybuf["wo"], None)], acts["att"], xf=xbuf["att"] if inq else None))
                if not inq:
                    quantize_x()
                # (the gate/up launch reads the rows of the down product after it ahead, as the decoder does)
                nxt = ([(L["down"], ybuf["down"], None)], False) if inq else None
                tm.launch("glu", wbytes["gate"] + wbytes["up"] + D + 4 * FFN,
                          lambda: dense.glu_mul(dev, L["gate"], L["up"], acts["x"], ybuf["gate"], xf=xf, norm=norm, ahead=nxt))
                if inq:
                    tm.launch("down", wbytes["down"] + FFN + 4 * D, lambda: dense.mv_multi(dev, [(L["down"], ybuf["down"], None)], xf=xbuf["mid"]))
                else:
                    dense.quantize_act(dev, xbuf["mid"], acts["mid"])
                    tm.launch("down", wbytes["down"] + FFN + 4 * D, lambda: dense.cmat_mul(dev, L["down"], acts["mid"], ybuf["down"]))
            else:
                quantize_x()
                for name, qt, rows, cols, src in specs:
                    if name == "wo":
                        dense.quantize_act(dev, xbuf["att"], acts["att"])
                    if name == "gate":
                        quantize_x()
                    if name == "down":
                        dense.quantize_act(dev, xbuf["mid"], acts["mid"])
                    tm.launch(name, wbytes[name] + cols + 4 * rows, lambda: dense.cmat_mul(dev, L[name], acts[src], ybuf[name]))
        if inq:
            tm.launch("head", head_host.size + D + 4 * VOCAB, lambda: dense.mv_multi(dev, [(head, logits, None)], xf=xbuf["x"], norm=norm))
        else:
            quantize_x()
            tm.launch("head", head_host.size + D + 4 * VOCAB, lambda: dense.cmat_mul(dev, head, acts["x"], logits))

    ms, dev_ms, per = tm.run(step, args.steps, args.warmup)
    # the roofline entry is the product kernel over all its launches of a step (one kernel, several shapes)
    allk = [sum(v[0] for v in per.values()), sum(v[1] for v in per.values()), sum(v[2] for v in per.values())]
    timed_by = "an event pair around every launch (the extra pass)"
    if inq:
        # The step is nothing but that kernel's launches, back to back on one stream: their average
        # duration is the timed steps' device time (the events around them) over their number.  The
        # extra pass's event pair per launch adds about 2 us to each and stays in by_launch_shape.
        nprobe = per["head"][2]
        allk = [dev_ms, allk[1] / nprobe, allk[2] // nprobe]
        timed_by = "the events around the timed steps: device_ms_per_step / launches per step"
    shapes = {k: {"GB/s": round(v[1] / (v[0] * 1e-3) / 1e9, 1), "avg_launch_us": round(v[0] / v[2] * 1e3, 2),
                  "bytes_per_launch": v[1] // v[2]} for k, v in per.items()}
    roof = roofline_of({"gemv": allk}, "hbm", HBM_PEAK_GBS, "GB/s",
                       {"gemv": "gemv_stream_kernel<12|14|0> (decode product, a workgroup's rows streamed into LDS: Q4_K, Q6_K, the mixed Q4_K+Q6_K launch; "
                                "gemv_kernel<FMT> where a product does not fit that way)"})
    roof["timed_by"] = timed_by
    roof["by_launch_shape"] = shapes
    roof["traffic"] = traffic_of("c2", per) if (args.mode in ("fused", "device") and nl == LAYERS) else None
    gbs = step_bytes / (ms * 1e-3) / 1e9

    def cpu():
        import oracle_lib as orc
        cores = host_cores()
        xs = {k: synth.activations(n, synth.make_rng(7)) for k, n in xin.items()}
        nbytes, t_cpu, reps = 0, 0.0, 0
        while t_cpu < 10.0 and reps < 4000:
            for name, qt, rows, cols, src in specs:
                t1 = time.perf_counter()
                orc.matmul(qt, host[name], rows, cols, xs[src], nthreads=cores)
                t_cpu += time.perf_counter() - t1
                nbytes += host[name].size
            reps += 1
        def one(nt):
            name, qt, rows, cols, src = specs[4]             # the gate matrix, 9728 x 2560 Q4_K
            orc.matmul(qt, host[name], rows, cols, xs[src], nthreads=nt)
            return host[name].size
        return {"value": round(nbytes / t_cpu / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
                "sample": f"{reps} x one layer's seven products (activation quantization included), {nbytes} weight bytes, {t_cpu:.1f} s",
                "tok_per_s_equiv": round(nbytes / t_cpu / step_bytes, 3),
                "one_thread": {"value": round(one_thread_figure(one) / 1e9, 3), "unit": "GB/s", "sample": "the 9728 x 2560 Q4_K product, about 3 s"}}

    return {"value": round(gbs, 1), "unit": "GB/s", "ms_per_step": ms, "device_ms_per_step": dev_ms, "enqueue_ms": tm.enqueue_ms,
            "dtype": "int8 block dots, fp32 combine",
            "config": {"workload": f"c2: qwen3-4b-shape decode, the {nl * 7 + 1} quantized matvecs of one token "
                                   f"({nl} layers x 7 + output head), Q4_K/Q6_K, batch 1",
                       "bytes_per_step": step_bytes, "layers": nl, "launch_mode": args.mode, "norms_included": bool(args.norm)},
            "extra": {"pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2), "matvec_only_tok_per_s": round(1e3 / ms, 1)},
            "roofline": roof, "cpu": cpu}


def workload_c1(args, dev):
    from illatio_amd import dense, hip, synth
    rng = synth.make_rng(11)
    shapes = [("up", 4864, 896), ("down", 896, 4864)]
    host = {n: synth.weights(synth.Q8_0, r, c, rng, dscale=0.02) for n, r, c in shapes}
    ncopy = 64
    mats = [{n: dense.upload_gmat(dev, n, synth.Q8_0, r, c, host[n]) for n, r, c in shapes} for _ in range(ncopy)]
    xs = {n: synth.activations(c, rng) for n, r, c in shapes}
    xb = {n: hip.hip_upload_new(dev, xs[n]) for n in xs}
    ys = {n: hip.hip_alloc(dev, 4 * r) for n, r, c in shapes}
    nbytes = {n: host[n].size + c // 32 * 34 + 4 * r for n, r, c in shapes}
    step_bytes = sum(host[n].size for n in host)
    tm = Timer(dev)

    def step(i):
        m = mats[i % ncopy]
        for n, r, c in shapes:      # the activation quantizer runs inside the product kernel
            tm.launch(n, nbytes[n], lambda: dense.mv_multi(dev, [(m[n], ys[n], None)], xf=xb[n]))

    ms, dev_ms, per = tm.run(step, args.steps, args.warmup, probe_steps=20)
    # the step is nothing but the product kernel's launches: their average duration from the events around the timed steps
    nprobe = per[shapes[0][0]][2]
    roof = roofline_of({"gemv": [dev_ms, sum(v[1] for v in per.values()) / nprobe, sum(v[2] for v in per.values()) // nprobe]},
                       "hbm", HBM_PEAK_GBS, "GB/s", {"gemv": "gemv_stream_kernel<8> (Q8_0 decode product, activations quantized in the kernel)"})
    roof["timed_by"] = "the events around the timed steps: device_ms_per_step / launches per step"
    roof["by_launch_shape"] = {k: {"avg_launch_us": round(v[0] / v[2] * 1e3, 2), "bytes_per_launch": v[1] // v[2]} for k, v in per.items()}
    roof["traffic"] = traffic_of("c1", per)
    gbs = step_bytes / (ms * 1e-3) / 1e9
    # the same two products on one copy of the matrices every step: 9 MB, in the memory-side cache (and mostly the L2s) after the first
    tc = Timer(dev)
    ms_cached, _, _ = tc.run(lambda i: [tc.launch(n, nbytes[n], lambda n=n: dense.mv_multi(dev, [(mats[0][n], ys[n], None)], xf=xb[n])) for n, r, c in shapes],
                             args.steps, args.warmup, probe_steps=0)

    def cpu():
        import oracle_lib as orc
        cores = host_cores()
        nb, t_cpu, reps = 0, 0.0, 0
        while t_cpu < 10.0 and reps < 20000:
            for n, r, c in shapes:
                t1 = time.perf_counter()
                orc.matmul(synth.Q8_0, host[n], r, c, xs[n], nthreads=cores)
                t_cpu += time.perf_counter() - t1
                nb += host[n].size
            reps += 1
        def one(nt):
            done = 0
            for n, r, c in shapes:
                orc.matmul(synth.Q8_0, host[n], r, c, xs[n], nthreads=nt)
                done += host[n].size
            return done
        return {"value": round(nb / t_cpu / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
                "sample": f"{reps} x both products (quantization included), {nb} weight bytes, {t_cpu:.1f} s",
                "one_thread": {"value": round(one_thread_figure(one) / 1e9, 3), "unit": "GB/s", "sample": "both products, about 3 s"}}

    return {"value": round(gbs, 1), "unit": "GB/s", "ms_per_step": ms, "device_ms_per_step": dev_ms, "enqueue_ms": tm.enqueue_ms, "dtype": "int8 block dots, fp32 combine",
            "config": {"workload": "c1: Q8_0 decode GEMV 4864x896 and 896x4864 (Qwen2-0.5B MLP), batch 1, rotating over 64 copies",
                       "bytes_per_step": step_bytes},
            "extra": {"pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
                      "cached_GBps": round(step_bytes / (ms_cached * 1e-3) / 1e9, 1)}, "roofline": roof, "cpu": cpu}


def workload_c3(args, dev):
    from illatio_amd import dense, hip, synth
    rng = synth.make_rng(33)
    rows, cols, T = (17408, 5120, args.tokens) if not args.transpose else (5120, 17408, args.tokens)
    # the benchmark's configuration 3 is Q6_K; --qtype: the same shape in the other dense formats (q8_0: the exact path only)
    qt = {"q4_k": synth.Q4_K, "q6_k": synth.Q6_K, "q8_0": synth.Q8_0}[args.qtype]
    if qt == synth.Q8_0 and args.path != "int8":
        raise SystemExit("bench.py: --qtype q8_0 goes with --path int8 (the bf16 product multiplies the K-quants)")
    w = np.tile(synth.weights(qt, 256, cols, rng, dscale=0.01), (rows // 256, 1))
    m = dense.upload_gmat(dev, "w", qt, rows, cols, w)
    x = synth.activations((T, cols), rng)
    xf = hip.hip_upload_new(dev, x)
    y = hip.hip_alloc(dev, 4 * T * rows, zero=False)
    flops = 2.0 * rows * cols * T
    tm = Timer(dev)
    bf16_path = args.path.startswith("bf16")
    path = args.path
    if path == "bf16":                           # the faster way from the quantized matrix: two passes pay from about a thousand tokens on
        path = "bf16-2pass" if T >= 1536 else "bf16-1pass"
    if path in ("bf16-2pass", "bf16-resident"):
        # the matrix dequantized to a bf16 copy (inside every step, or once beforehand and kept), then the plain bf16 product
        xb = hip.hip_alloc(dev, dense.slabs_bytes(T, cols), zero=False)
        wb = dense.dequant_bf16(dev, m)
        resident = path == "bf16-resident"

        def step(_):
            tm.launch("cvt", 0, lambda: dense.cvt_bf16_slabs(dev, xf, T, cols, xb))
            if not resident:
                tm.launch("dequant", 0, lambda: dense.dequant_bf16(dev, m, wb))
            tm.launch("mm", flops, lambda: dense.mat_mul_bf16(dev, wb, rows, cols, xb, y, T))
        names = {"mm": "gemm_bf16_plain_kernel (both operands bf16 through LDS, v_mfma_f32_32x32x16_bf16)"}
    elif path == "bf16-1pass":
        xb = hip.hip_alloc(dev, 2 * T * cols, zero=False)

        def step(_):
            tm.launch("cvt", 0, lambda: dense.cvt_bf16(dev, xf, T * cols, xb))
            tm.launch("mm", flops, lambda: dense.cmat_mul_bf16(dev, m, xb, y, T))
        names = {"mm": "gemm_bf16_kernel<14, TM, TN, NB> (Q6_K dequantized to bf16 in LDS, v_mfma_f32_32x32x16_bf16)"}
    elif path in ("int8-2pass", "int8-resident"):
        # the exact product from the two int8 planes of the matrix, written inside every step or once beforehand and kept
        act = dense.QAct(dev, T, cols, ("q8k",))
        planes = dense.planes_i8(dev, m)
        resident = path == "int8-resident"

        def step(_):
            tm.launch("quant", 0, lambda: dense.quantize_act(dev, xf, act))
            if not resident:
                tm.launch("planes", 0, lambda: dense.planes_i8(dev, m, planes))
            tm.launch("mm", flops, lambda: dense.mat_mul_i8_planes(dev, planes, rows, cols, act, y, T))
        names = {"mm": "gemm_i8pp_kernel (the two int8 planes of scale * (quant - 32) read as they were written beforehand, v_mfma_i32_32x32x32_i8, "
                       "one float combine per super-block: bit-exact with the CPU path)"}
    else:
        act = dense.QAct(dev, T, cols, ("q8",) if qt == synth.Q8_0 else ("q8k",))

        def step(_):
            tm.launch("quant", 0, lambda: dense.quantize_act(dev, xf, act))
            tm.launch("mm", flops, lambda: dense.cmat_mul(dev, m, act, y, n=T))
        names = {"mm": "gemm_i8p_kernel (scale * quant as two int8 planes in LDS, v_mfma_i32_32x32x32_i8, one float combine per super-block: "
                       "bit-exact with the CPU path)"}
    ms, dev_ms, per = tm.run(step, args.steps, args.warmup)
    roof = roofline_of({k: v for k, v in per.items() if k == "mm"}, "mfma", MFMA_PEAK_TFLOPS[args.path], "TFLOP/s" if bf16_path else "TOP/s", names)
    roof["unit"] = "TFLOP/s"
    if path in TRAFFIC.get("c3", {}) and T == 4096 and not args.transpose and args.qtype == "q6_k":
        roof["traffic"] = TRAFFIC["c3"][path]
    tf = flops / (ms * 1e-3) / 1e12

    def cpu():
        import oracle_lib as orc
        cores = host_cores()
        ts = 16
        t1 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t1 < 10.0:
            orc.matmul(qt, w, rows, cols, x[:ts], nthreads=cores)
            reps += 1
        t_cpu = time.perf_counter() - t1
        def one(nt):
            orc.matmul(qt, w, rows, cols, x[:1], nthreads=nt)
            return 2.0 * rows * cols
        return {"value": round(2.0 * rows * cols * ts * reps / t_cpu / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
                "sample": f"{reps} x the same matrix on {ts} tokens (quantization included), {t_cpu:.1f} s",
                "one_thread": {"value": round(one_thread_figure(one) / 1e12, 5), "unit": "TFLOP/s", "sample": "the same matrix on one token, about 3 s"}}

    return {"value": round(tf, 1), "unit": "TFLOP/s", "ms_per_step": ms, "device_ms_per_step": dev_ms, "enqueue_ms": tm.enqueue_ms,
            "dtype": "bf16 x bf16, fp32 accumulate" if bf16_path else "int8 block dots, fp32 combine",
            "metric": "prefill product TFLOP/s (% of dense MFMA peak)",
            "config": {"workload": f"c3: {args.qtype.upper()} prefill product {rows}x{cols} on {T} tokens, {path} path "
                                   f"(activation conversion inside the step)", "flops_per_step": flops, "tokens": T},
            "extra": {"pct_of_mfma_peak": round(100 * tf / MFMA_PEAK_TFLOPS[args.path], 2),
                      # the step's algorithmic bytes (the quantized matrix once, the float activations, the float results) over its
                      # time: far below 8,000 GB/s, i.e. not bound by memory at this token count
                      "algorithmic_GBps": round((w.size + 4.0 * T * cols + 4.0 * T * rows) / (ms * 1e-3) / 1e9, 1)},
            "roofline": roof, "cpu": cpu}


def moe_weights(rng, ne_unique, ne, d, ff):
    from illatio_amd import synth
    reps = ne // ne_unique
    gate = np.tile(synth.weights(synth.IQ2_XXS, ne_unique * ff, d, rng), (reps, 1))
    up = np.tile(synth.weights(synth.IQ2_XXS, ne_unique * ff, d, rng), (reps, 1))
    down = np.tile(synth.weights(synth.Q2_K, ne_unique * d, ff, rng), (reps, 1))
    return gate, up, down


def workload_c4(args, dev):
    from illatio_amd import ds4f, hip, synth
    rng = synth.make_rng(44)
    ne, nu, d, ff, nlayers = 256, 6, 4096, 2048, 3
    gate, up, down = moe_weights(rng, 32, ne, d, ff)
    sg, su = (synth.weights(synth.Q8_0, ff, d, rng) for _ in range(2))
    sd = synth.weights(synth.Q8_0, d, ff, rng)
    pools = [ds4f.ExpertPool(dev, ne, d, ff, gate, up, down) for _ in range(nlayers)]
    shared = [ds4f.SharedExpert(dev, d, ff, sg, su, sd) for _ in range(nlayers)]
    x = synth.activations(d, rng)
    xb = hip.hip_upload_new(dev, x)
    nsteps = args.steps + args.warmup + 12
    tables, routes = [], []
    fused, ondev = args.mode == "fused", args.mode == "device"
    logits = []
    for i in range(nsteps):                      # the reference routes on the CPU (cuda-ds4f.lisp:991-999); tables made beforehand
        lg = synth.activations(ne, rng)
        lgb = hip.hip_upload_new(dev, lg)
        if ondev:                                # device mode: only the router's logits are resident; d4_route runs in the step
            logits.append(lgb)
            routes.append(None)
        else:                                    # the tables of the host-routed modes, made by d4_route ahead of the timed steps
            dsel, dw = ds4f.route(dev, lgb, 1, ne, nu, 1.5)
            sel, w = hip.hip_download(dsel, np.uint32, nu).astype(np.int32), hip.hip_floats(dw, nu)
            for b in (lgb, dsel, dw):
                hip.hip_free(b)
            routes.append((sel, w))
            tables.append((ds4f.fused_tables if fused else ds4f.tail_tables)(dev, pools[i % nlayers], sel, w))
    ws = hip.Workspace(dev, 8 << 20)
    step_ws = hip.hip_alloc(dev, ds4f.step_workspace_bytes(nu, d, ff), zero=False)
    moe_out = hip.hip_alloc(dev, 4 * d)
    iq, q2, q8 = synth.row_bytes(synth.IQ2_XXS, d), synth.row_bytes(synth.Q2_K, ff), 34
    step_bytes = nu * (2 * ff * iq + d * q2) + 2 * ff * d // 32 * q8 + d * ff // 32 * q8
    tm = Timer(dev)

    def step(i):
        ws.reset()
        L = i % nlayers
        sel, w = routes[i] if routes[i] else (None, None)
        if ondev and not tm.probing:             # the step as one call into the library (the routing rides along with the shared expert's gate/up launch, the sum with its down launch: 4 launches)
            ds4f.ffn_step_call(dev, pools[L], shared[L], logits[i], xb, moe_out, ne, nu, 1.5, 0.0, wsbuf=step_ws)
        elif ondev:                              # the probing pass: the same kernels launched one by one (6 launches), an event pair around each
            ds4f.ffn_step_device(dev, pools[L], shared[L], logits[i], xb, ne, nu, 1.5, 0.0, ws=ws)
        elif fused:
            ds4f.ffn_step_fused(dev, pools[L], shared[L], sel, w, xb, 0.0, ws=ws, tables=tables[i])
        else:
            ds4f.ffn_tail(dev, pools[L], sel, w, xb, ds4f.ffn_shared(dev, shared[L], xb, 0.0, ws=ws), 0.0, ws=ws, tables=tables[i])

    def work_of(kernel, a):          # weight bytes + quantized activations + float outputs of the product kernels
        if kernel in ("d4_mv_iq2_xxs", "d4_mv_glu_iq2_xxs"):
            return 2 * nu * ff * iq + d + d // 256 * 4 + 4 * 2 * nu * ff
        if kernel in ("d4_mv_q2_k", "d4_mv_q2_k_f32"):
            return nu * (d * q2 + ff + ff // 256 * 4 + ff // 16 * 4) + 4 * nu * d
        if kernel == "d4_mvq8":
            return a[0] * a[1] // 32 * q8 + a[1] // 32 * 36 + 4 * a[0]
        if kernel == "d4_mvq8_glu":
            return 2 * a[0] * a[1] // 32 * q8 + a[1] // 32 * 36 + 4 * a[0]
        return 0

    ms, dev_ms, per = tm.run(step, args.steps, args.warmup, probe_steps=10, work_of=work_of)
    if ondev:
        # the timed sequence itself (four launches queued by one call), the library recording an event before each of
        # its launches and one behind the last: per launch, the median over 20 steps
        import ctypes as C
        evs = [hip.hip_event_create(dev, True) for _ in range(5)]
        arr = (C.c_uint64 * 5)(*evs)
        hip.call("ilt_d4_ffn_step_events", arr, C.c_int(5))
        gaps = []
        try:
            for i in range(20):
                ds4f.ffn_step_call(dev, pools[i % nlayers], shared[i % nlayers], logits[i % len(logits)], xb, moe_out, ne, nu, 1.5, 0.0, wsbuf=step_ws)
                hip.hip_sync(dev)
                gaps.append([hip.hip_event_elapsed_ms(evs[k], evs[k + 1]) for k in range(4)])
        finally:
            hip.call("ilt_d4_ffn_step_events", None, C.c_int(0))
        for e in evs:
            hip.hip_event_destroy(e)
        med = np.median(np.array(gaps), axis=0)
        names = ["d4_mvq8_glu+route", "d4_mv_glu_iq2_xxs", "d4_mv_q2_k_f32", "d4_mvq8+sum"]
        works = [work_of("d4_mvq8_glu", [ff, d]), work_of("d4_mv_glu_iq2_xxs", None), work_of("d4_mv_q2_k_f32", None), work_of("d4_mvq8", [d, ff])]
        per = {nm: [float(med[k]), works[k], 1] for k, nm in enumerate(names)}
    roof = roofline_of({k: v for k, v in per.items() if v[1]}, "hbm", HBM_PEAK_GBS, "GB/s",
                       {"d4_mvq8_glu+route": "gemv_stream_kernel<8, 0> (shared expert's Q8_0 gate, up and gated activation; one of its waves routes the token)",
                        "d4_mvq8+sum": "gemv_stream_kernel<8, 2> (shared expert's Q8_0 down, the step's ordered sum carried along)",
                        "d4_mv_glu_iq2_xxs": "gemv_stream_kernel<16, 0> (the 6 selected experts' IQ2_XXS gate, up and gated activation, one launch)",
                        "d4_mv_q2_k_f32": "gemv_stream_kernel<10, 0> (the 6 selected experts' Q2_K down)"} if ondev else
                       {"d4_mv_iq2_xxs": "gemv_kernel<16> (the 6 selected experts' IQ2_XXS gate and up, one launch over 12 matrices)",
                        "d4_mv_glu_iq2_xxs": "gemv_kernel<16> (the 6 selected experts' IQ2_XXS gate, up and gated activation, one launch)",
                        "d4_mv_q2_k": "gemv_kernel<10> (the 6 experts' Q2_K down)", "d4_mv_q2_k_f32": "gemv_kernel<10> (the 6 experts' Q2_K down)",
                        "d4_mvq8": "gemv_kernel<8> (shared expert, Q8_0)", "d4_mvq8_glu": "gemv_kernel<8> (shared expert gate, up, gated activation)"})
    roof["launch_us_all"] = {k: round(v[0] / v[2] * 1e3, 2) for k, v in per.items()}
    dom = max((k for k in per if per[k][1]), key=lambda k: per[k][0])
    roof["traffic"] = TRAFFIC.get("c4", {}).get(dom)
    if ondev:
        roof["timed_by"] = "events the library records around each launch of the timed one-call step (an event pair adds about 2 us to a launch)"
    gbs = step_bytes / (ms * 1e-3) / 1e9

    def cpu():
        import oracle_lib as orc
        cores = host_cores()
        crng = synth.make_rng(45)
        t1, reps = time.perf_counter(), 0
        while time.perf_counter() - t1 < 10.0:
            sel, w = orc.route(synth.activations(ne, crng), nu, 1.5)
            orc.moe_routed(gate, up, down, d, ff, sel, w, 0.0, x, nthreads=cores)
            orc.moe_shared(sg, su, sd, d, ff, 0.0, x, nthreads=cores)
            reps += 1
        t_cpu = time.perf_counter() - t1
        def one(nt):
            sel, w = orc.route(synth.activations(ne, crng), nu, 1.5)
            orc.moe_routed(gate, up, down, d, ff, sel, w, 0.0, x, nthreads=nt)
            orc.moe_shared(sg, su, sd, d, ff, 0.0, x, nthreads=nt)
            return step_bytes
        return {"value": round(step_bytes * reps / t_cpu / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
                "sample": f"{reps} decode steps (6 routed experts + shared expert), {t_cpu:.1f} s",
                "one_thread": {"value": round(one_thread_figure(one) / 1e9, 3), "unit": "GB/s", "sample": "the same steps, about 3 s"}}

    return {"value": round(gbs, 1), "unit": "GB/s", "ms_per_step": ms, "device_ms_per_step": dev_ms, "enqueue_ms": tm.enqueue_ms, "dtype": "int8 block dots, fp32 combine",
            "metric": "MoE decode step achieved HBM GB/s (% of 8 TB/s)",
            "config": {"workload": f"c4: MoE decode step, 256 resident experts (IQ2_XXS gate/up, Q2_K down) top-6 + Q8_0 shared expert, "
                                   f"d 4096, ff 2048, batch 1, rotating over {nlayers} layers", "bytes_per_step": step_bytes},
            "extra": {"pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2), "launches_per_step": 4 if ondev else 5 if fused else 12,
                      "launch_mode": args.mode}, "roofline": roof, "cpu": cpu}


def workload_c5(args, dev):
    from illatio_amd import ds4f, hip, synth
    rng = synth.make_rng(55)
    ne, nu, d, ff, n = 256, 6, 4096, 2048, args.tokens
    gate, up, down = moe_weights(rng, 32, ne, d, ff)
    pool = ds4f.ExpertPool(dev, ne, d, ff, gate, up, down)
    norms = synth.activations((n, d), rng)
    logits = synth.zipf_router_logits(n, ne, rng)
    lb, nb = hip.hip_upload_new(dev, logits), hip.hip_upload_new(dev, norms)
    sb = hip.hip_alloc(dev, 4 * n * d)           # the rows the ordered sum ends with, zeros: configuration 5 states no shared expert (a chunk's
                                                 # shared expert is ffn_shared_chunk's, timed with the decode step's in c4)
    rows = n * nu
    ws = hip.Workspace(dev, rows * (4 * d * 2 + 2 * d + 4 * ff * 3 + 2 * ff + d + ff + 4096) + 4 * n * d + (16 << 20))
    flops = 2.0 * rows * 3 * ff * d
    tm = Timer(dev)
    fn = ds4f.ffn_routed_chunk_bf16 if args.path == "bf16" else ds4f.ffn_routed_chunk

    def step(_):
        ws.reset()
        fn(dev, pool, lb, nb, sb, n, ne, nu, 1.5, 0.0, ws=ws)

    def work_of(kernel, a):
        if kernel == "d4_mm_id_bf16":
            return 2.0 * rows * a[1] * a[2]
        if kernel == "d4_mm_id_glu_bf16":            # gate and up
            return 2 * 2.0 * rows * a[1] * a[2]
        if kernel in ("d4_mm_id_iq2_xxs", "d4_mm_id_q2_k"):
            return 2.0 * rows * a[0] * a[1]
        return 0

    ms, dev_ms, per = tm.run(step, args.steps, args.warmup, probe_steps=2, work_of=work_of)
    # the grouped products: gate + up (IQ2_XXS; one launch with the gated activation on the bf16 path) and down (Q2_K)
    mm = [k for k in per if per[k][1]]
    allmm = [sum(per[k][0] for k in mm), sum(per[k][1] for k in mm), sum(per[k][2] for k in mm)]
    roof = roofline_of({"mm_id": allmm}, "mfma", MFMA_PEAK_TFLOPS[args.path], "TFLOP/s",
                       {"mm_id": "gemm_bf16_regb_kernel<16, true> (d4_mm_id_glu_bf16: gate, up, activation) + <10, false> (d4_mm_id_bf16: down)" if args.path == "bf16"
                        else "gemm_i8p_kernel<16> (d4_mm_id_iq2_xxs x2) + <10> (d4_mm_id_q2_k): scale * quant as int8 planes, grouped, bit-exact with the CPU path"})
    roof["launch_us_all"] = {k: round(v[0] / v[2] * 1e3, 2) for k, v in per.items()}
    if args.path == "bf16" and n == 4096:
        t5 = TRAFFIC.get("c5", {})
        roof["traffic"] = int(sum(t5.values()) / len(t5)) if t5 else None       # per launch, over the step's two grouped launches
    tf = flops / (ms * 1e-3) / 1e12

    def cpu():
        import oracle_lib as orc
        cores = host_cores()
        ts = 8
        t1, reps = time.perf_counter(), 0
        while time.perf_counter() - t1 < 10.0:
            orc.moe_chunk(gate, up, down, d, ff, ne, nu, 1.5, 0.0, logits[:ts], norms[:ts], None, nthreads=cores)
            reps += 1
        t_cpu = time.perf_counter() - t1
        def one(nt):
            orc.moe_chunk(gate, up, down, d, ff, ne, nu, 1.5, 0.0, logits[:1], norms[:1], None, nthreads=nt)
            return 2.0 * nu * 3 * ff * d
        return {"value": round(2.0 * ts * nu * 3 * ff * d * reps / t_cpu / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
                "sample": f"{reps} chunks of {ts} tokens (48 rows each), {t_cpu:.1f} s",
                "one_thread": {"value": round(one_thread_figure(one) / 1e12, 5), "unit": "TFLOP/s", "sample": "one token's six experts, about 3 s"}}

    return {"value": round(tf, 1), "unit": "TFLOP/s", "ms_per_step": ms, "device_ms_per_step": dev_ms, "enqueue_ms": tm.enqueue_ms,
            "dtype": "bf16 x bf16, fp32 accumulate" if args.path == "bf16" else "int8 block dots, fp32 combine",
            "metric": "MoE prefill grouped product TFLOP/s (% of dense MFMA peak)",
            "config": {"workload": f"c5: MoE prefill chunk, {n} tokens x top-6 of 256 experts (Zipf 1.1), IQ2_XXS gate/up, Q2_K down, "
                                   f"d 4096, ff 2048, {args.path} path, routing to ordered sum", "flops_per_step": flops, "tokens": n},
            "extra": {"pct_of_mfma_peak": round(100 * tf / MFMA_PEAK_TFLOPS[args.path], 2),
                      # the chunk's algorithmic bytes (every expert's matrices once, the tokens' rows in, the summed rows out)
                      # over its time: not bound by memory
                      "algorithmic_GBps": round((ne * (2.0 * pool.gate_bytes + pool.down_bytes) + 2 * 4.0 * n * d) / (ms * 1e-3) / 1e9, 1)},
            "roofline": roof, "cpu": cpu}


def workload_c2d(args, dev):
    """Config 2 as it is stated: the whole dense decoder at the Qwen3-4B shape (36 layers, head norms, RoPE,
    grouped-query attention over an fp32 KV cache, Q4_K / Q6_K weights), random-init: a 512-token prompt through the
    prefill products, then a 256-token greedy decode at batch 1.  A step is one decoded token: its whole forward pass to
    the logits and the greedy pick -- on the device, the ids read back after the last token (--host-argmax: logits
    downloaded and the token picked on the host every step, as the reference's loop does, cuda-dense.lisp:428-430)."""
    from illatio_amd import hip, model, synth
    q8 = getattr(args, "q8_model", False)                    # c1d: config 1's family (Qwen2.5-0.5B's shape, Q8_0, 24 layers)
    nl, nprompt, ndecode = (min(args.layers, 24) if q8 else args.layers), 512, 256
    host = model.synth_model_q8(2, nl=nl) if q8 else model.synth_model(2, nl=nl)
    shape = "qwen2.5-0.5b" if q8 else "qwen3-4b"
    c = host["config"]
    m = model.DenseModel(dev, host, nctx=nprompt + ndecode + args.warmup + 8, chunk=512)
    rng = synth.make_rng(3)
    prompt = rng.integers(0, c["vocab"], nprompt).tolist()
    m.eval_tokens(prompt)                                    # once untimed: the first launch of each kernel
    m.reset()
    hip.hip_sync(dev)
    t0 = time.perf_counter()
    m.eval_tokens(prompt)
    hip.hip_sync(dev)
    prefill_s = time.perf_counter() - t0
    tok = m.argmax()
    for _ in range(args.warmup):
        m.forward_n([tok]); tok = m.argmax()
    hip.hip_sync(dev)
    t0 = time.perf_counter()
    if args.host_argmax:                                     # the reference's loop: logits to the host, the token picked there
        toks = []
        for _ in range(ndecode):
            m.forward_n([tok])
            tok = m.argmax()
            toks.append(tok)
    else:                                                    # the token picked on the device and fed on from device memory
        toks = m.decode_greedy(ndecode)
    hip.hip_sync(dev)
    decode_s = time.perf_counter() - t0
    wbytes = sum(a[1].size for L in host["layers"] for k, a in L.items() if isinstance(a, tuple)) + host["output"][1].size
    ms = decode_s * 1e3 / ndecode
    m.free()
    more = {}
    if not q8:
        # the same prompt through the bf16 matrix-core products (on the CPU path's quantized activations; within the
        # bf16 roundings of the exact prefill, not equal to it), from the quantized matrices and from bf16 copies kept resident
        for mode in ("bf16", "bf16-resident"):
            mb = model.DenseModel(dev, host, nctx=nprompt + 8, chunk=512, prefill=mode)
            mb.eval_tokens(prompt)
            mb.reset()
            hip.hip_sync(dev)
            t0 = time.perf_counter()
            mb.eval_tokens(prompt)
            hip.hip_sync(dev)
            more[f"prefill_{mode.replace('-', '_')}_tok_per_s"] = round(nprompt / (time.perf_counter() - t0), 1)
            mb.free()
        # the decode at a context past the one-launch attention's 1,024 positions: a 2,048-token prompt, 64 greedy tokens
        ml = model.DenseModel(dev, host, nctx=2048 + 64 + 8)      # (the prompt in one chunk)
        long_prompt = rng.integers(0, c["vocab"], 2048).tolist()
        ml.eval_tokens(long_prompt)
        ml.reset()
        hip.hip_sync(dev)
        t0 = time.perf_counter()
        ml.eval_tokens(long_prompt)
        hip.hip_sync(dev)
        more["prefill_tok_per_s_2048_token_prompt"] = round(2048 / (time.perf_counter() - t0), 1)
        ml.decode_greedy(4)
        hip.hip_sync(dev)
        t0 = time.perf_counter()
        ml.decode_greedy(60)
        hip.hip_sync(dev)
        more["decode_tok_per_s_at_2048_positions"] = round(60 / (time.perf_counter() - t0), 1)
        ml.free()

    def cpu():
        import oracle_lib as orc
        cores = host_cores()
        cm = orc.DenseModel(host, 64)
        t_tok = prompt[0]
        cm.forward(t_tok, nthreads=cores)                     # the pool's threads started, the weights touched
        t1 = time.perf_counter()
        n = 0
        while time.perf_counter() - t1 < 10.0 and n < 60:
            logits, _ = cm.forward(t_tok, nthreads=cores)
            t_tok = int(np.argmax(logits))
            n += 1
        t_cpu = time.perf_counter() - t1
        t2 = time.perf_counter()
        cm.forward(t_tok, nthreads=1)
        one = 1.0 / (time.perf_counter() - t2)
        return {"value": round(n / t_cpu, 3), "unit": "tok/s", "cores": cores, "kind": "port",
                "sample": f"{n} greedy tokens of the same model from an empty context (attention over at most {n + 1} positions), {t_cpu:.1f} s",
                "one_thread": {"value": round(one, 3), "unit": "tok/s", "sample": "one more token on one thread"}}

    return {"value": round(ndecode / decode_s, 1), "unit": "tok/s", "ms_per_step": ms, "device_ms_per_step": ms, "enqueue_ms": 0.0,
            "dtype": "int8 block dots, fp32 combine; fp32 attention",
            "metric": "decode tok/s at Qwen2.5-0.5B shape" if q8 else "decode tok/s at Qwen3-4B shape",
            "config": {"workload": f"{'c1' if q8 else 'c2'} decode: {shape}-shape dense decoder, {nl} layers, random-init {'Q8_0' if q8 else 'Q4_K/Q6_K'}, {nprompt}-token prompt then "
                                   f"{ndecode}-token greedy decode at batch 1", "weight_bytes_per_token": int(wbytes)},
            "extra": {"prefill_tok_per_s": round(nprompt / prefill_s, 1), "distinct_tokens_decoded": len(set(toks)), "tokens_decoded": ndecode,
                      "weights_GBps_in_decode": round(wbytes / (ms * 1e-3) / 1e9, 1), **more},
            "roofline": {"bound": "hbm", "achieved": round(wbytes / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(wbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                         "kernel": "whole token: 5 launches a layer (Q/K/V, attention, wo, gate+up, down) + embedding + head + the "
                                   "greedy pick's two",
                         "launches": 5 * nl + 4, "avg_launch_us": round(ms * 1e3 / (5 * nl + 4), 2)},
            "cpu": cpu}


def workload_c1d(args, dev):
    """Config 1's family as a whole decoder: the Qwen2.5-0.5B shape in Q8_0 (24 layers, hidden 896, intermediate 4864, 14
    query heads on 2 KV heads of 64, biases on Q, K and V), random-init: a 512-token prompt, then 256 greedy tokens."""
    import copy
    a = copy.copy(args)
    a.q8_model = True
    return workload_c2d(a, dev)


WORKLOADS = {"c1": workload_c1, "c1d": workload_c1d, "c2": workload_c2, "c2d": workload_c2d, "c3": workload_c3, "c4": workload_c4, "c5": workload_c5}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS),
                    help="one workload only; default: c2 (the line's value) and then c1, c3, c4, c5 under \"configs\"")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--layers", type=int, default=LAYERS, help=argparse.SUPPRESS)
    ap.add_argument("--tokens", type=int, default=4096, help="c3, c5: tokens per step")
    ap.add_argument("--transpose", action="store_true", help="c3: the 5120x17408 matrix")
    ap.add_argument("--host-argmax", action="store_true", help="c2d: every token's logits to the host and the next token picked there")
    ap.add_argument("--qtype", default="q6_k", choices=["q6_k", "q4_k", "q8_0"], help="c3: the matrix's format (the benchmark's: q6_k)")
    ap.add_argument("--path", default="bf16", choices=["bf16", "bf16-1pass", "bf16-2pass", "bf16-resident", "int8", "int8-2pass", "int8-resident"],
                    help="c3, c5: which matrix-core path.  c3: bf16 = 2pass from 1536 tokens on, else 1pass; bf16-1pass = the matrix dequantized inside the product's loop; "
                         "bf16-2pass = the matrix dequantized to a bf16 copy inside the step, then the plain bf16 product; bf16-resident = that copy made beforehand and kept")
    ap.add_argument("--norm", action="store_true", help="c2: include each layer's two norms and the output norm (inside the product launches in fused mode)")
    ap.add_argument("--mode", default="fused", choices=["fused", "fused-q", "single", "device"],
                    help="c4: fused = 5 launches a step, single = the reference's sequence of 12 (both with the routing done beforehand on the host, as the "
                         "reference routes on the CPU), device = the routing inside the step (carried along by the shared expert's gate/up launch), the expert kernels indexing the slot table by its result, one call into the library (5 launches).  c2: fused = Q/K/V in one launch, gate+up in one, activations quantized inside the product "
                         "kernels; fused-q = the same launches after separate quantizer launches; "
                         "single = one launch per matrix after separate quantizer launches")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N above 1 is not supported "
              "(the path would shard by rows of a matrix and by experts; nothing here uses a second GPU)", file=sys.stderr)
        return 2

    from illatio_amd import hip
    dev = hip.open_hip(0)
    everything = args.workload is None
    if everything:
        args.workload = "c2"
    r = WORKLOADS[args.workload](args, dev)
    out = {"metric": r.get("metric", "Q-matvec achieved HBM GB/s (% of 8 TB/s); decode tok/s at Qwen3-4B shape"),
           "value": r["value"], "unit": r["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(r["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": r["dtype"], "data": "synthetic", "config": r["config"]}
    out.update(r["extra"])
    out["device_ms_per_step"] = round(r["device_ms_per_step"], 4)
    out["host_enqueue_ms_per_step"] = round(r["enqueue_ms"], 4)
    out["roofline"] = r["roofline"]
    out["cpu_baseline"] = None if args.no_cpu else r["cpu"]()
    if everything:
        # the benchmark's other configurations on the same clock (no CPU leg): c4 with the routing on the device, c3 and
        # c5 on the bf16 matrix cores at 4096 tokens and, as a second entry each, on the bit-exact int8 path; c3 also at
        # its other two token counts and with the matrix's bf16 copy made once and kept (2 bytes a weight of the 288 GB)
        import copy
        import gc
        out["configs"] = {}
        extras = [("c2_decode", {}), ("c1", {"steps": 200, "warmup": 20}), ("c1_decode", {}), ("c3", {"path": "bf16", "tokens": 4096}), ("c3_t2048", {"path": "bf16", "tokens": 2048}),
                  ("c3_t512", {"path": "bf16", "tokens": 512}), ("c3_resident", {"path": "bf16-resident", "tokens": 4096}),
                  ("c3_exact", {"path": "int8", "tokens": 4096}),
                  ("c4", {"mode": "device", "steps": 50, "warmup": 5}), ("c5", {"path": "bf16", "tokens": 4096}), ("c5_exact", {"path": "int8", "tokens": 4096})]
        for name, over in extras:
            a = copy.copy(args)
            a.workload, a.steps, a.warmup = {"c2_decode": "c2d", "c1_decode": "c1d"}.get(name, name[:2]), min(args.steps, 10), min(args.warmup, 3)
            for k, v in over.items():
                setattr(a, k, v)
            del r
            gc.collect()
            r = WORKLOADS[a.workload](a, dev)
            roof = r["roofline"]
            if name == "c2_decode":
                out["decode_tok_per_s"] = r["value"]
                out["decode_ms_per_token"] = round(r["ms_per_step"], 4)
                out["prefill_tok_per_s"] = r["extra"]["prefill_tok_per_s"]
            out["configs"][name] = {
                "workload": r["config"]["workload"], "value": r["value"], "unit": r["unit"], "ms_per_step": round(r["ms_per_step"], 4),
                "steps": r["extra"].get("tokens_decoded", a.steps), "warmup": a.warmup, "dtype": r["dtype"], "extra": r["extra"],
                "roofline": {k: roof.get(k) for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "launches", "avg_launch_us",
                                                      "launch_us_all", "other_kernels")}}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
