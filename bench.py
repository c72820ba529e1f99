#!/usr/bin/env python3
"""Headline benchmark: the Qwen3.5-2B-like decode matvec set on one MI355X.

A step is one pass of the decode set at N = 1 token: attention_in [q|k|v], mixer_out
[o], ffn_in [gate|up] (Q4_K), ffn_down (Q6_K) and the 151,936-row lm_head (Q6_K),
285.6 MB of packed weights, issued in decode order on one stream as one recorded
graph.  Inputs and weights are resident in HBM before the timed region.  Steps
rotate over distinct copies of the weights so that no step finds its weights in the
256 MB last-level cache.

Prints one JSON line: value = weight bytes per second over the whole set, roofline =
the dominant kernel (the Q6_K lm_head GEMV) against the 8 TB/s HBM peak, timed live
with HIP events on the library's stream, and cpu_baseline = the same set on the
host's cores through the reference's own CPU code (or its C restatement).
"""
from __future__ import annotations

import argparse
import json
import sys
import time

import numpy as np

import __graft_entry__ as entry

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0  # dense fp16 / bf16
# HBM bytes one lm_head launch moves, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
# (`bench.py --counters`), each scaled by what the same counter reads for the 256 MiB
# read / write probe: 255,449,700 fetched + 613,867 written, 1.0008 x the algorithmic
# 255,868,416.  Counters cannot be read from inside this process; re-measure with the
# two commands in profiles/kquant_gemv_decode_set_hbm_traffic.md after a kernel change.
LM_HEAD_TRAFFIC_BYTES = 256063566


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--lm-head-copies", type=int, default=3)
    ap.add_argument("--layer-copies", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--details", action="store_true",
                    help="also time every stage and the other configurations (stderr)")
    ap.add_argument("--counters", action="store_true",
                    help="for a `rocprofv3 --pmc` run: a few plain launches of every decode "
                         "stage plus the read and write probes (known byte counts that "
                         "calibrate the memory counters), no timing")
    ap.add_argument("--prefill-counters", action="store_true",
                    help="for a `rocprofv3` run: a few plain launches of the prefill GEMM "
                         "(config 5), no timing")
    return ap.parse_args()


def run_prefill_counters(capi, cfg, synth, launches=6):
    """Plain launches of the config-5 GEMM for a trace or counter run."""
    spec = cfg.CONFIG5
    mw = capi.Matrix(spec.ggml_type, spec.build(), spec.rows, spec.cols)
    a_bits = synth.bf16_round(synth.activations(cfg.CONFIG5_TOKENS, spec.cols, cfg.CONFIG5_A_SEED))
    da = capi.DeviceBuffer.from_array(a_bits)
    dc = capi.DeviceBuffer(4 * cfg.CONFIG5_TOKENS * spec.rows)
    for _ in range(launches):
        capi.gemm_q4k_bf16_dev(mw, da, cfg.CONFIG5_TOKENS, dc)
        capi.synchronize()
    # and as many with the weights prepared once: the pre-pass then converts activations only
    mw.prepare_prefill()
    for _ in range(launches):
        capi.gemm_q4k_bf16_dev(mw, da, cfg.CONFIG5_TOKENS, dc)
        capi.synchronize()
    print(json.dumps({"prefill_counters_run": {
        "launches": launches, "launches_prepared": launches,
        "tokens": cfg.CONFIG5_TOKENS, "rows": spec.rows, "cols": spec.cols,
        "flops_per_launch": 2 * cfg.CONFIG5_TOKENS * spec.rows * spec.cols}}))


def run_counters(capi, cfg, decode):
    """Plain (unrecorded) launches, so that a counter run attributes every dispatch."""
    window = 256 << 20
    buf = capi.DeviceBuffer(window)
    sink = capi.DeviceBuffer(64)
    for _ in range(3):
        capi.write_probe_dev(buf, window)
    for _ in range(3):
        capi.read_probe_dev(buf, window, sink)
    capi.synchronize()
    for stage in cfg.CONFIG2_STAGES:
        for i in range(6):
            decode.stage(stage, i)
    capi.synchronize()
    print(json.dumps({"counters_run": {"probe_bytes": window,
                                       "launches_per_stage": 6,
                                       "stages": list(cfg.CONFIG2_STAGES)}}))


def log(*args):
    print(*args, file=sys.stderr, flush=True)


class DecodeSet:
    """Device-resident copies of the config-2 matrices and the stage calls."""

    def __init__(self, capi, cfg, synth, layer_copies, head_copies):
        self.capi, self.cfg = capi, cfg
        self.host = {name: spec.build() for name, spec in cfg.CONFIG2.items()}
        self.layers = []
        for _ in range(layer_copies):
            self.layers.append({n: capi.Matrix(s.ggml_type, self.host[n], s.rows, s.cols)
                                for n, s in cfg.CONFIG2.items() if n != "lm_head"})
        head = cfg.CONFIG2["lm_head"]
        self.heads = [capi.Matrix(head.ggml_type, self.host["lm_head"], head.rows, head.cols)
                      for _ in range(head_copies)]
        self.x_host = synth.activations(1, cfg.HIDDEN2, cfg.CONFIG2_X_SEED)
        self.act_host = synth.activations(1, cfg.FFN2, cfg.CONFIG2_ACT_SEED)
        self.x = capi.DeviceBuffer.from_array(self.x_host)
        self.act = capi.DeviceBuffer.from_array(self.act_host)
        self.out = {stage: capi.DeviceBuffer(4 * sum(cfg.CONFIG2[n].rows for n in names))
                    for stage, names in cfg.CONFIG2_STAGES.items()}

    def stage(self, stage, copy):
        capi, cfg = self.capi, self.cfg
        if stage == "lm_head":
            mats = [self.heads[copy % len(self.heads)]]
        else:
            layer = self.layers[copy % len(self.layers)]
            mats = [layer[n] for n in cfg.CONFIG2_STAGES[stage]]
        x = self.act if stage == "ffn_down" else self.x
        capi.gemv_dev([capi.whole(m) for m in mats], x, 1, self.out[stage])

    def fused_stage(self, stage, copy):
        """The stage with the elementwise step Decoder::Step runs before it taken into
        the product: residual add + RmsNorm before attention_in, ffn_in and lm_head,
        SwiGLU before ffn_down (which then reads ffn_in's [gate | up] row)."""
        capi, cfg = self.capi, self.cfg
        if not hasattr(self, "norm"):
            import numpy as np
            self.norm = capi.DeviceBuffer.from_array(np.ones(cfg.HIDDEN2, dtype=np.float32))
            self.residual = [capi.DeviceBuffer(4 * cfg.HIDDEN2) for _ in range(3)]
        if stage == "lm_head":
            mats = [self.heads[copy % len(self.heads)]]
        else:
            layer = self.layers[copy % len(self.layers)]
            mats = [layer[n] for n in cfg.CONFIG2_STAGES[stage]]
        parts = [capi.whole(m) for m in mats]
        if stage == "mixer_out":
            capi.gemv_dev(parts, self.x, 1, self.out[stage])
        elif stage == "ffn_down":
            capi.gemv_fused_dev(parts, capi.swiglu_prologue(), self.out["ffn_in"], 1,
                                self.out[stage])
        else:
            slot = {"attention_in": 0, "ffn_in": 1, "lm_head": 2}[stage]
            delta = self.out["ffn_down" if slot != 1 else "mixer_out"]
            prologue = capi.resnorm_prologue(self.norm, 1e-6, delta, self.residual[slot])
            capi.gemv_fused_dev(parts, prologue, self.x, 1, self.out[stage])

    def step(self, copy):
        for stage in self.cfg.CONFIG2_STAGES:
            self.stage(stage, copy)

    def record(self, copy):
        self.capi.capture_begin()
        self.step(copy)
        return self.capi.capture_end()


def time_graphs(capi, graphs, steps, warmup):
    for i in range(warmup):
        graphs[i % len(graphs)].launch()
    capi.synchronize()
    capi.timer_begin()
    for i in range(steps):
        graphs[(warmup + i) % len(graphs)].launch()
    ms = capi.timer_end()
    capi.synchronize()
    return ms / steps


def time_calls(capi, call, steps, warmup):
    for i in range(warmup):
        call(i)
    capi.synchronize()
    capi.timer_begin()
    for i in range(steps):
        call(warmup + i)
    ms = capi.timer_end()
    capi.synchronize()
    return ms / steps


def time_recorded(capi, calls, reps=20, warmup=3):
    """Per-call time of `calls` (a list of thunks that enqueue _dev products):
    recorded once as one graph and replayed, so host enqueue cost stays out."""
    for call in calls:  # an ordinary pass first: recording cannot allocate scratch
        call()
    capi.synchronize()
    capi.capture_begin()
    for call in calls:
        call()
    graph = capi.capture_end()
    for _ in range(warmup):
        graph.launch()
    capi.synchronize()
    capi.timer_begin()
    for _ in range(reps):
        graph.launch()
    ms = capi.timer_end()
    capi.synchronize()
    graph.destroy()
    return ms / (reps * len(calls))


def report(name, nbytes, ms, extra=""):
    log(f"  {name:34s} {nbytes / 1e6:8.2f} MB  {ms * 1e3:8.2f} us  {nbytes / ms / 1e6:8.1f} GB/s"
        f"  {100 * nbytes / ms / 1e6 / HBM_PEAK_GBS:5.1f}% of peak {extra}")


def run_details(capi, cfg, synth, decode, args):
    """Every stage of the decode set and the other measured configurations, each
    rotating over enough weight copies to stay out of the 256 MB last-level cache."""
    import numpy as np

    log("config 2, per stage (N=1):")
    for stage, names in cfg.CONFIG2_STAGES.items():
        nbytes = sum(cfg.CONFIG2[n].nbytes for n in names)
        n = 6 if stage == "lm_head" else 30
        ms = time_recorded(capi, [lambda i=i, s=stage: decode.stage(s, i) for i in range(n)])
        report(stage, nbytes, ms)

    log("config 2, the same stages with the decoder's elementwise steps inside the product "
        "(residual add + RmsNorm before attention_in / ffn_in / lm_head, SwiGLU before "
        "ffn_down):")
    fused_total = 0.0
    for stage, names in cfg.CONFIG2_STAGES.items():
        nbytes = sum(cfg.CONFIG2[n].nbytes for n in names)
        n = 6 if stage == "lm_head" else 30
        ms = time_recorded(capi, [lambda i=i, s=stage: decode.fused_stage(s, i)
                                  for i in range(n)])
        fused_total += ms
        report(stage + (" (plain)" if stage == "mixer_out" else " (fused)"), nbytes, ms)
    log(f"  sum of the five stages with the steps inside: {fused_total * 1e3:.2f} us")

    log("config 2, greedy decoding: the head product and the pick of its first maximum:")
    index = capi.DeviceBuffer(8)
    head_bytes = cfg.CONFIG2["lm_head"].nbytes
    ms_head = time_recorded(capi, [lambda i=i: decode.stage("lm_head", i) for i in range(6)])
    capi.synchronize()
    # The separate pick copies its result to the host, which a recording cannot hold:
    # timed from the host, launch and copy latency included.
    reps = 50
    start = time.perf_counter()
    for _ in range(reps):
        capi.argmax_dev(decode.out["lm_head"], cfg.CONFIG2["lm_head"].rows)
    ms_pick_sync = (time.perf_counter() - start) * 1e3 / reps
    ms_fused = time_recorded(capi, [lambda i=i: capi.gemv_argmax_dev(
        [capi.whole(decode.heads[i % len(decode.heads)])], None, decode.x, 1, index)
        for i in range(6)])
    report("lm_head, logits stored", head_bytes, ms_head)
    log(f"    + separate pick over the stored logits (2 launches, result copied to the host, "
        f"synchronous): {ms_pick_sync * 1e3:.1f} us")
    report("lm_head with the pick inside", head_bytes, ms_fused)
    index.free()

    log("read probe (plain streaming read, the ceiling a kernel can reach):")
    probe = capi.DeviceBuffer(1 << 30)
    sink = capi.DeviceBuffer(64)
    window = 256 << 20
    ms = time_recorded(capi, [lambda i=i: capi.read_probe_dev_at(probe, (i % 4) * window, window,
                                                                 sink) for i in range(8)])
    report("read probe 256 MiB", window, ms)
    probe.free()

    log("config 1, single Q4_K GEMV 6144x2048 (N=1), 40 weight copies:")
    spec = cfg.CONFIG1
    host = spec.build()
    mats = [capi.Matrix(spec.ggml_type, host, spec.rows, spec.cols) for _ in range(40)]
    x = capi.DeviceBuffer.from_array(synth.activations(1, spec.cols, cfg.CONFIG1_X_SEED))
    y = capi.DeviceBuffer(4 * spec.rows)
    ms = time_recorded(capi, [lambda m=m: capi.gemv_dev([capi.whole(m)], x, 1, y) for m in mats])
    report("q4_k 6144x2048 from HBM", spec.nbytes, ms)
    ms = time_recorded(capi, [lambda: capi.gemv_dev([capi.whole(mats[0])], x, 1, y)] * 40)
    report("q4_k 6144x2048 cache resident", spec.nbytes, ms)
    for m in mats:
        m.destroy()

    log("other row types of real files (not in the configurations), N=1, 40 copies from HBM:")
    for name, ggml_type, rows, cols in (("q8_0 2048x2048", synth.Q8_0, 2048, 2048),
                                        ("f32 router 257x2048", synth.F32, 257, 2048)):
        host = synth.matrix(ggml_type, rows, cols, 7)
        mats = [capi.Matrix(ggml_type, host, rows, cols) for _ in range(40)]
        y2 = capi.DeviceBuffer(4 * rows)
        ms = time_recorded(capi, [lambda m=m: capi.gemv_dev([capi.whole(m)], x, 1, y2)
                                  for m in mats])
        report(name, host.size, ms)
        for m in mats:
            m.destroy()
        y2.free()

    log("config 3, MTP-verify FFN (gate|up 9216x2560 Q4_K, down 2560x9216 Q6_K), 8 copies:")
    gate, up, down = (cfg.CONFIG3[n] for n in ("gate", "up", "down"))
    hg, hu, hd = gate.build(), up.build(), down.build()
    sets = [(capi.Matrix(gate.ggml_type, hg, gate.rows, gate.cols),
             capi.Matrix(up.ggml_type, hu, up.rows, up.cols),
             capi.Matrix(down.ggml_type, hd, down.rows, down.cols)) for _ in range(8)]
    base = {}
    for tokens in (1, 2, 3, 4):
        xin = capi.DeviceBuffer.from_array(synth.activations(tokens, cfg.HIDDEN3, 1))
        act = capi.DeviceBuffer.from_array(synth.activations(tokens, cfg.FFN3, 2))
        y_in = capi.DeviceBuffer(4 * tokens * 2 * cfg.FFN3)
        y_down = capi.DeviceBuffer(4 * tokens * cfg.HIDDEN3)
        ms_in = time_recorded(capi, [lambda s=s: capi.gemv_dev([capi.whole(s[0]), capi.whole(s[1])],
                                                               xin, tokens, y_in) for s in sets])
        ms_down = time_recorded(capi, [lambda s=s: capi.gemv_dev([capi.whole(s[2])], act, tokens,
                                                                 y_down) for s in sets])
        if tokens == 1:
            base = {"in": ms_in, "down": ms_down}
        report(f"gate|up N={tokens}", gate.nbytes + up.nbytes, ms_in,
               f"x{ms_in / base['in']:.2f} of N=1")
        report(f"down    N={tokens}", down.nbytes, ms_down, f"x{ms_down / base['down']:.2f} of N=1")
        for b in (xin, act, y_in, y_down):
            b.free()
    for s in sets:
        for m in s:
            m.destroy()

    log("config 5, prefill projection (4096 x 2048 bf16 activations . Q4_K 6144 x 2048):")
    spec = cfg.CONFIG5
    mw = capi.Matrix(spec.ggml_type, spec.build(), spec.rows, spec.cols)
    a_bits = synth.bf16_round(synth.activations(cfg.CONFIG5_TOKENS, spec.cols, cfg.CONFIG5_A_SEED))
    da = capi.DeviceBuffer.from_array(a_bits)
    dc = capi.DeviceBuffer(4 * cfg.CONFIG5_TOKENS * spec.rows)
    ms = time_recorded(capi, [lambda: capi.gemm_q4k_bf16_dev(mw, da, cfg.CONFIG5_TOKENS, dc)] * 4,
                       reps=10)
    flops = 2.0 * cfg.CONFIG5_TOKENS * spec.rows * spec.cols
    log(f"  gemm 4096x6144x2048 (pre-pass + MFMA kernel)  {ms * 1e3:8.2f} us  "
        f"{flops / ms / 1e9:8.1f} TFLOP/s  {100 * flops / ms / 1e9 / MFMA_PEAK_TFLOPS:5.1f}% of "
        f"the {MFMA_PEAK_TFLOPS:.0f} TFLOP/s fp16/bf16 peak")
    mw.prepare_prefill()  # the fp16 weights stay with the matrix: 25 MB beside its 7 MB
    ms = time_recorded(capi, [lambda: capi.gemm_q4k_bf16_dev(mw, da, cfg.CONFIG5_TOKENS, dc)] * 4,
                       reps=10)
    log(f"  the same, weights prepared once beforehand      {ms * 1e3:8.2f} us  "
        f"{flops / ms / 1e9:8.1f} TFLOP/s  {100 * flops / ms / 1e9 / MFMA_PEAK_TFLOPS:5.1f}%")
    mw.destroy()
    da.free()
    dc.free()

    log("config 4, MoE experts (256 experts, hidden 2048, ffn 512, top-8):")
    gate, up, down = (cfg.CONFIG4[n] for n in ("gate", "up", "down"))
    mg = capi.Matrix(gate.ggml_type, gate.build(), gate.rows, gate.cols)
    mu = capi.Matrix(up.ggml_type, up.build(), up.rows, up.cols)
    md = capi.Matrix(down.ggml_type, down.build(), down.rows, down.cols)
    per_expert = (gate.nbytes + up.nbytes + down.nbytes) // cfg.EXPERTS4
    for tokens in (1, 4):
        calls, distinct = [], []
        keep = []
        for r in range(16):  # 16 different routings, so successive calls read other experts
            logits = synth.router_logits(tokens, cfg.EXPERTS4, 900 + 16 * tokens + r)
            xh = synth.activations(tokens, cfg.HIDDEN4, 950 + r) * np.float32(cfg.CONFIG4_X_SCALE)
            dl = capi.DeviceBuffer.from_array(logits)
            dx = capi.DeviceBuffer.from_array(xh)
            ids = capi.DeviceBuffer(4 * tokens * cfg.TOPK4)
            wts = capi.DeviceBuffer(4 * tokens * cfg.TOPK4)
            yo = capi.DeviceBuffer(4 * tokens * cfg.HIDDEN4)
            keep += [dl, dx, ids, wts, yo]
            host_ids, _ = capi.route_topk(logits, cfg.TOPK4)
            distinct.append(len(set(host_ids.reshape(-1).tolist())))

            def call(dl=dl, dx=dx, ids=ids, wts=wts, yo=yo):
                capi.route_topk_dev(dl, tokens, cfg.EXPERTS4, cfg.TOPK4, ids, wts)
                capi.moe_ffn_dev(mg, mu, md, cfg.EXPERTS4, dx, tokens, ids, wts, cfg.TOPK4, yo)
            calls.append(call)
        ms = time_recorded(capi, calls)
        mean_distinct = sum(distinct) / len(distinct)
        report(f"route+group+experts batch {tokens}", int(mean_distinct * per_expert), ms,
               f"({mean_distinct:.1f} distinct experts; kernels: route, "
               f"{'' if tokens == 1 else 'group, '}gate|up, down, combine)")
        for b in keep:
            b.free()
    # The whole layer in one call: router product (F32, 256 + 1 rows), routing, experts, and
    # the shared expert's rows scaled by the sigmoid of the extra logit.
    router = capi.Matrix(synth.F32, synth.f32_matrix(cfg.EXPERTS4 + 1, cfg.HIDDEN4, 990),
                         cfg.EXPERTS4 + 1, cfg.HIDDEN4)
    for tokens in (1, 4):
        calls, keep = [], []
        for r in range(16):
            xh = synth.activations(tokens, cfg.HIDDEN4, 960 + r) * np.float32(cfg.CONFIG4_X_SCALE)
            dx = capi.DeviceBuffer.from_array(xh)
            shared = capi.DeviceBuffer.from_array(synth.activations(tokens, cfg.HIDDEN4, 970 + r))
            yo = capi.DeviceBuffer(4 * tokens * cfg.HIDDEN4)
            keep += [dx, shared, yo]
            calls.append(lambda dx=dx, shared=shared, yo=yo: capi.moe_layer_dev(
                router, mg, mu, md, cfg.EXPERTS4, cfg.TOPK4, dx, tokens, shared, yo))
        ms = time_recorded(capi, calls)
        log(f"  whole layer in one call, batch {tokens}                 {ms * 1e3:8.2f} us  "
            f"(router product + the kernels above + the scaled shared expert in the combine)")
        for b in keep:
            b.free()
    for m in (mg, mu, md, router):
        m.destroy()


def cpu_baseline(cfg, decode, seconds):
    """The same set on the host cores: the reference's fused AVX2 dots on its own
    thread pool (oracle/_ref), or the scalar C restatement where that is absent."""
    oracle = entry.load_oracle()
    use_ref = oracle.ref_available()
    if use_ref:
        threads = oracle.ref().ref_default_threads()
        kind = "reference"
    else:
        import os
        threads = max(len(os.sched_getaffinity(0)) // 2, 1)
        kind = "port"
    stages = []
    for stage, names in cfg.CONFIG2_STAGES.items():
        parts = [(cfg.CONFIG2[n].ggml_type, decode.host[n], 0, cfg.CONFIG2[n].rows)
                 for n in names]
        stages.append((parts, decode.act_host if stage == "ffn_down" else decode.x_host))

    def one_set():
        for parts, x in stages:
            oracle.matmul(parts, x, threads=threads, use_ref=use_ref)

    one_set()  # warm the pool and the page tables
    t0 = time.perf_counter()
    one_set()
    probe = time.perf_counter() - t0
    reps = int(max(3, min(5000, seconds / max(probe, 1e-6))))
    t0 = time.perf_counter()
    for _ in range(reps):
        one_set()
    elapsed = time.perf_counter() - t0
    per_set = elapsed / reps
    gbs = cfg.config2_bytes() / per_set / 1e9
    what = ("gguf_dot AVX2 dots on the reference's SpinPool" if use_ref
            else "scalar C restatement, pthreads")
    return {"value": round(gbs, 3), "unit": "GB/s", "cores": threads, "kind": kind,
            "sample": f"{reps} passes of the full 285.6 MB decode set ({what}), "
                      f"{per_set * 1e3:.2f} ms per set"}


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only; rerun with --gpus 1 "
              "(each box has one GPU and the path needs no collective)", file=sys.stderr)
        sys.exit(2)
    entry.load_package()
    from gufo_npu_amd import capi, configs as cfg, synth

    capi.init(0)
    device, cus = capi.device_info()
    log(f"device: {device}, {cus} CUs")
    if args.prefill_counters:
        run_prefill_counters(capi, cfg, synth)
        return
    t0 = time.perf_counter()
    decode = DecodeSet(capi, cfg, synth, args.layer_copies, args.lm_head_copies)
    log(f"weights resident: {args.layer_copies} layer copies, {args.lm_head_copies} "
        f"lm_head copies ({time.perf_counter() - t0:.1f} s)")

    if args.counters:
        run_counters(capi, cfg, decode)
        return

    set_bytes = cfg.config2_bytes()
    n_graphs = max(args.layer_copies, args.lm_head_copies)
    n_graphs = args.layer_copies * args.lm_head_copies // np.gcd(args.layer_copies,
                                                                 args.lm_head_copies)
    n_graphs = min(n_graphs, 30)
    decode.step(0)
    capi.synchronize()
    graphs = [decode.record(i) for i in range(n_graphs)]

    # The timed region: exactly `steps` decode sets after `warmup` untimed ones.
    capi.synchronize()
    ms_step = time_graphs(capi, graphs, args.steps, args.warmup)
    value = set_bytes / (ms_step * 1e-3) / 1e9

    # Dominant kernel: the lm_head GEMV, back to back over the rotating copies.
    head = cfg.CONFIG2["lm_head"]
    head_bytes = head.nbytes + 4 * (head.cols + head.rows)
    ms_head = time_calls(capi, lambda i: decode.stage("lm_head", i), args.steps, args.warmup)
    achieved = head_bytes / (ms_head * 1e-3) / 1e9

    result = {
        "metric": "K-quant GEMV HBM GB/s (% of peak) + µs per decode-token matvec set, 1 GPU",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "Qwen3.5-2B-like decode matvec set, N=1: q 2048x2048, k/v 512x2048, "
                        "o 2048x2048, gate/up 6144x2048 (Q4_K), down 2048x6144 (Q6_K), "
                        "lm_head 151936x2048 (Q6_K); x fp32 N(0,1)",
            "weight_bytes_per_step": set_bytes,
            "us_per_set": round(ms_step * 1e3, 3),
            "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
            "launches_per_step": len(cfg.CONFIG2_STAGES),
            "weight_copies": {"layer": args.layer_copies, "lm_head": args.lm_head_copies},
            "device": device,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "KquantGemvKernel<Q6_K, N=1> (lm_head 151936x2048)",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "us_per_launch": round(ms_head * 1e3, 3),
            "bytes_per_launch": head_bytes,
            "traffic": LM_HEAD_TRAFFIC_BYTES,
        },
    }

    if args.details:
        run_details(capi, cfg, synth, decode, args)

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(cfg, decode, args.cpu_seconds)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result, ensure_ascii=False))


if __name__ == "__main__":
    main()
