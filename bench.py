#!/usr/bin/env python3
"""bench.py -- the quantized matrix-product path on one MI355X.

A step is one decoded token's worth of quantized products at the Qwen3-4B shape
(BASELINE.json configs[1]): for each of 36 layers the activation quantizations and the
seven matrix-vector products (Q4_K wq 4096x2560, wk 1024x2560, wo 2560x4096, gate and up
9728x2560; Q6_K wv 1024x2560, down 2560x9728), then the Q6_K output head 151936x2560 --
2,618,273,280 bytes of GGUF blocks streamed from HBM per step, every matrix its own
allocation, so the working set (2.6 GB) is far beyond the 256 MB MALL.  Weights and
activations are synthetic and seeded (illatio_amd/synth.py); inputs are resident in HBM
before the timed region.  No attention, norm or RoPE runs in a step: those belong to the
dense-forward harness, not to this path.

Prints one JSON line: metric "Q-matvec achieved HBM GB/s ...", value = GB/s of GGUF bytes
over the whole step, plus the roofline of the dominant kernel (timed with HIP events on the
launch stream in a second pass over the same sequence) and the CPU oracle timed on a
bounded sample of the same workload on this host.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0

D, FFN, QD, KVD, VOCAB, LAYERS = 2560, 9728, 4096, 1024, 151936, 36


def layer_matrices():
    from illatio_amd import synth
    return [("wq", synth.Q4_K, QD, D, "x"), ("wk", synth.Q4_K, KVD, D, "x"), ("wv", synth.Q6_K, KVD, D, "x"),
            ("wo", synth.Q4_K, D, QD, "att"), ("gate", synth.Q4_K, FFN, D, "x"), ("up", synth.Q4_K, FFN, D, "x"),
            ("down", synth.Q6_K, D, FFN, "mid")]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--layers", type=int, default=LAYERS, help=argparse.SUPPRESS)
    ap.add_argument("--mode", default="fused", choices=["fused", "fused-q", "single"],
                    help="fused: Q/K/V in one launch, gate+up in one, activations quantized inside the product "
                         "kernels; fused-q: the same launches after separate quantizer launches; "
                         "single: one launch per matrix after separate quantizer launches")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N above 1 is not supported "
              "(the path shards by rows / by experts, see DESIGN.md)", file=sys.stderr)
        return 2

    from illatio_amd import dense, hip, synth
    dev = hip.open_hip(0)
    rng = synth.make_rng(42)
    nl = args.layers

    # ---- weights: one seeded layer's bytes, uploaded to a separate allocation per layer ----
    specs = layer_matrices()
    host = {name: synth.weights(qt, rows, cols, rng) for name, qt, rows, cols, _ in specs}
    layers = []
    for li in range(nl):
        layers.append({name: dense.upload_gmat(dev, f"blk.{li}.{name}", qt, rows, cols, host[name])
                       for name, qt, rows, cols, _ in specs})
    head_host = synth.weights(synth.Q6_K, VOCAB, D, rng)
    head = dense.upload_gmat(dev, "output", synth.Q6_K, VOCAB, D, head_host)
    step_bytes = nl * sum(synth.row_bytes(qt, cols) * rows for _, qt, rows, cols, _ in specs) + head_host.size

    # ---- activations (device resident) ----
    xin = {"x": D, "att": QD, "mid": FFN}
    xbuf = {k: hip.hip_upload_new(dev, synth.activations(n, rng)) for k, n in xin.items()}
    acts = {k: dense.QAct(dev, 1, n, ("q8k",)) for k, n in xin.items()}
    ybuf = {name: hip.hip_alloc(dev, 4 * rows) for name, _, rows, _, _ in specs}
    logits = hip.hip_alloc(dev, 4 * VOCAB)

    ev = [hip.hip_event_create(dev, timing=True) for _ in range(2)]
    probes = []          # (kernel label, bytes, start event, stop event) when profiling

    wbytes = {name: synth.row_bytes(qt, cols) * rows for name, qt, rows, cols, _ in specs}

    def timed(fn, nbytes, probe):
        if probe:
            e0, e1 = hip.hip_event_create(dev, True), hip.hip_event_create(dev, True)
            hip.hip_event_record(e0, dev.stream)
        fn()
        if probe:
            hip.hip_event_record(e1, dev.stream)
            probes.append(("gemv_kernel", nbytes, e0, e1))

    fused, inq = args.mode != "single", args.mode == "fused"

    def step(probe=False):
        for L in layers:
            if fused:
                xf = xbuf["x"] if inq else None
                if not inq:
                    dense.quantize_act(dev, xbuf["x"], acts["x"])
                timed(lambda: dense.qkv_mul(dev, L["wq"], L["wk"], L["wv"], acts["x"], ybuf["wq"], ybuf["wk"], ybuf["wv"], xf=xf),
                      wbytes["wq"] + wbytes["wk"] + wbytes["wv"] + D + 4 * (QD + 2 * KVD), probe)
                if not inq:
                    dense.quantize_act(dev, xbuf["att"], acts["att"])
                timed(lambda: dense.mv_multi(dev, [(L["wo"], ybuf["wo"], None)], acts["att"], xf=xbuf["att"] if inq else None),
                      wbytes["wo"] + QD + 4 * D, probe)
                if not inq:
                    dense.quantize_act(dev, xbuf["x"], acts["x"])
                timed(lambda: dense.glu_mul(dev, L["gate"], L["up"], acts["x"], ybuf["gate"], xf=xf),
                      wbytes["gate"] + wbytes["up"] + D + 4 * FFN, probe)
                # the down projection's input is 9728 wide: quantized once, not by every workgroup
                dense.quantize_act(dev, xbuf["mid"], acts["mid"])
                timed(lambda: dense.cmat_mul(dev, L["down"], acts["mid"], ybuf["down"]), wbytes["down"] + FFN + 4 * D, probe)
            else:
                dense.quantize_act(dev, xbuf["x"], acts["x"])
                for name, qt, rows, cols, src in specs:
                    if name == "wo":
                        dense.quantize_act(dev, xbuf["att"], acts["att"])
                    if name == "gate":
                        dense.quantize_act(dev, xbuf["x"], acts["x"])
                    if name == "down":
                        dense.quantize_act(dev, xbuf["mid"], acts["mid"])
                    timed(lambda: dense.cmat_mul(dev, L[name], acts[src], ybuf[name]), wbytes[name] + cols + 4 * rows, probe)
        if inq:
            timed(lambda: dense.mv_multi(dev, [(head, logits, None)], xf=xbuf["x"]), head_host.size + D + 4 * VOCAB, probe)
        else:
            dense.quantize_act(dev, xbuf["x"], acts["x"])
            timed(lambda: dense.cmat_mul(dev, head, acts["x"], logits), head_host.size + D + 4 * VOCAB, probe)

    for _ in range(args.warmup):
        step()
    hip.hip_sync(dev)
    t0 = time.perf_counter()
    hip.hip_event_record(ev[0], dev.stream)
    for _ in range(args.steps):
        step()
    hip.hip_event_record(ev[1], dev.stream)
    hip.hip_sync(dev)
    wall_ms = (time.perf_counter() - t0) * 1e3
    dev_ms = hip.hip_event_elapsed_ms(ev[0], ev[1])
    ms_per_step = max(wall_ms, dev_ms) / args.steps
    gbs = step_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- roofline of the dominant kernel: HIP events around each launch, same sequence ----
    for _ in range(max(1, min(args.steps, 5))):
        step(probe=True)
    hip.hip_sync(dev)
    per = {}
    for label, nbytes, e0, e1 in probes:
        ms = hip.hip_event_elapsed_ms(e0, e1)
        t = per.setdefault(label, [0.0, 0, 0])
        t[0] += ms; t[1] += nbytes; t[2] += 1
        hip.hip_event_destroy(e0); hip.hip_event_destroy(e1)
    dom = max(per, key=lambda k: per[k][0])
    dms, dbytes, dn = per[dom]
    achieved = dbytes / (dms * 1e-3) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                "kernel": "gemv_kernel<0> (dense Q4_K/Q6_K decode product)", "launches": dn, "avg_launch_us": round(dms / dn * 1e3, 2),
                "avg_bytes_per_launch": dbytes // dn,
                "other_kernels": {k: {"GB/s": round(v[1] / (v[0] * 1e-3) / 1e9, 1), "launches": v[2]}
                                  for k, v in per.items() if k != dom}}

    # ---- CPU baseline: the oracle (a C restatement of the reference's CPU path) on this host ----
    cpu = None
    if not args.no_cpu:
        import oracle_lib as orc
        cores = min(os.cpu_count() or 1, 64)
        try:
            cores = min(cores, len(os.sched_getaffinity(0)))
        except AttributeError:
            pass
        xs = {k: synth.activations(n, synth.make_rng(7)) for k, n in xin.items()}
        sample_bytes, t_cpu, reps = 0, 0.0, 0
        while t_cpu < 10.0 and reps < 4000:
            for name, qt, rows, cols, src in specs:
                t1 = time.perf_counter()
                orc.matmul(qt, host[name], rows, cols, xs[src], nthreads=cores)
                t_cpu += time.perf_counter() - t1
                sample_bytes += host[name].size
            reps += 1
        cpu = {"value": round(sample_bytes / t_cpu / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": f"{reps} x one layer's seven products (activation quantization included), "
                         f"{sample_bytes} weight bytes, {t_cpu:.1f} s",
               "tok_per_s_equiv": round(sample_bytes / t_cpu / step_bytes, 3)}

    out = {"metric": "Q-matvec achieved HBM GB/s (% of 8 TB/s); decode tok/s at Qwen3-4B shape",
           "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "int8 block dots, fp32 combine", "data": "synthetic",
           "config": {"workload": f"qwen3-4b-shape decode: the {nl * 7 + 1} quantized matvecs of one token "
                                  f"({nl} layers x 7 + output head), Q4_K/Q6_K, batch 1",
                      "bytes_per_step": step_bytes, "layers": nl, "launch_mode": args.mode},
           "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
           "matvec_only_tok_per_s": round(1e3 / ms_per_step, 1),
           "device_ms_per_step": round(dev_ms / args.steps, 4),
           "roofline": roofline, "cpu_baseline": cpu}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
