#!/usr/bin/env python3
"""Benchmark of the quantized matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--sweep]

A step is one launch of the hot kernel over one batch of synthetic input: by
default the Q4 batch-1 GEMV at the Llama-3-8B FFN shape W[4096,14336] (the
configuration the headline metric is quoted on).  Steps rotate through enough
distinct copies of the weight (>= 512 MiB) that no step finds its weight in a
cache: the figure is an HBM figure.  Inputs are resident in HBM before the
timed region; the region is bracketed by HIP events recorded on the stream the
kernels run on, with a device synchronisation on both sides.

Timing method (examples/matmul_throughput.rs:114-127 is the model): the weight
copies are created and touched, the device is pre-heated with at least 100 ms
of launches, `--warmup` further untimed steps follow, then `--steps` launches
are timed `--repeats` times (at least 5); `ms_per_step` is the median repeat,
the fastest and slowest are reported beside it.  The same line carries, under
`configs`, every BASELINE workload timed the same way (200 launches per
repeat, median of 5).

Prints ONE JSON line on stdout.  `--sweep` additionally measures the cache-warm
figures and the quantizers and writes the table to stderr and, with
`--sweep-out FILE`, as JSON to that file.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, vendor figure
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense fp16 MFMA, vendor figure

Q4, Q8 = 0, 1

# name: (fmt, m, k, n, residual, fp16 activations, BASELINE config index)
WORKLOADS = {
    "c5_q4_m1_4096x14336": (Q4, 1, 4096, 14336, False, False, 5),
    "c5_q4_m1_14336x4096": (Q4, 1, 14336, 4096, False, False, 5),
    "c5_q8_m1_4096x14336": (Q8, 1, 4096, 14336, False, False, 5),
    "c5_q8_m1_14336x4096": (Q8, 1, 14336, 4096, False, False, 5),
    "c5_q4_m4_4096x14336": (Q4, 4, 4096, 14336, False, False, 5),
    "c5_q4_m16_4096x14336": (Q4, 16, 4096, 14336, False, False, 5),
    "c5_q8_m4_4096x14336": (Q8, 4, 4096, 14336, False, False, 5),
    "c5_q8_m16_4096x14336": (Q8, 16, 4096, 14336, False, False, 5),
    "c5_q4_m4_14336x4096": (Q4, 4, 14336, 4096, False, False, 5),
    "c5_q4_m16_14336x4096": (Q4, 16, 14336, 4096, False, False, 5),
    "c5_q8_m4_14336x4096": (Q8, 4, 14336, 4096, False, False, 5),
    "c5_q8_m16_14336x4096": (Q8, 16, 14336, 4096, False, False, 5),
    "c3_q4_lm_head_576x49152": (Q4, 1, 576, 49152, False, False, 3),
    "c1_q8_up_576x1536": (Q8, 1, 576, 1536, False, False, 1),
    "c2_q4_q_576x576": (Q4, 1, 576, 576, False, False, 2),
    "c2_q4_kv_576x192": (Q4, 1, 576, 192, False, False, 2),
    "c2_q4_o_576x576_add": (Q4, 1, 576, 576, True, False, 2),
    "c2_q4_gate_up_576x3072": (Q4, 1, 576, 3072, False, False, 2),
    "c2_q4_down_1536x576_add": (Q4, 1, 1536, 576, True, False, 2),
    "c4_q4_prefill_up_512x1024x3072": (Q4, 512, 1024, 3072, False, True, 4),
    "c4_q4_prefill_down_512x3072x1024": (Q4, 512, 3072, 1024, False, True, 4),
    # C4 with the f32 activations the reference's Session hands to a matmul (BASELINE names fp16)
    "c4_f32a_q4_prefill_up_512x1024x3072": (Q4, 512, 1024, 3072, False, False, 4),
    "c4_f32a_q4_prefill_down_512x3072x1024": (Q4, 512, 3072, 1024, False, False, 4),
    # not a BASELINE configuration: four times the headline weight, to separate the kernel's
    # streaming rate from the fixed cost of a launch (sweep only)
    "scale_q4_m1_8192x28672": (Q4, 1, 8192, 28672, False, False, 5),
}
HEADLINE = "c5_q4_m1_4096x14336"

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the
# same counters read for a 256 MiB device copy (one summary per workload under profiles/).
MEASURED_TRAFFIC_BYTES = {
    "c5_q4_m1_4096x14336": 37.02e6,
    "c5_q4_m1_14336x4096": 37.42e6,
    "c5_q8_m1_4096x14336": 63.57e6,
    "c5_q8_m1_14336x4096": 64.02e6,
    "c5_q4_m4_4096x14336": 37.71e6,
    "c5_q4_m4_14336x4096": 39.55e6,
    "c5_q8_m4_4096x14336": 64.56e6,
    "c5_q8_m4_14336x4096": 66.31e6,
    "c5_q4_m16_4096x14336": 50.11e6,
    "c5_q4_m16_14336x4096": 56.63e6,
    "c5_q8_m16_4096x14336": 74.80e6,
    "c5_q8_m16_14336x4096": 82.33e6,
    "c3_q4_lm_head_576x49152": 18.02e6,
    "c1_q8_up_576x1536": 1.17e6,
    "c2_q4_gate_up_576x3072": 1.33e6,
    "c2_q4_down_1536x576_add": 0.74e6,
    "c2_q4_q_576x576": 0.39e6,
    "c4_q4_prefill_up_512x1024x3072": 19.00e6,
    "c4_q4_prefill_down_512x3072x1024": 32.97e6,
    "c4_f32a_q4_prefill_up_512x1024x3072": 27.29e6,
    "c4_f32a_q4_prefill_down_512x3072x1024": 37.60e6,
}


def algorithmic_bytes(fmt, m, k, n, resid, f16):
    """Bytes one call must move: packed weight once (20 B per Q4 block; 34 B per Q8
    block, the reference's 2 pad bytes are not credited), activations, output
    (and the residual when there is one)."""
    blocks = (k // 32) * n
    wbytes = blocks * (20 if fmt == Q4 else 34)
    return wbytes + (2 if f16 else 4) * m * k + 4 * m * n * (2 if resid else 1)


class WeightSets:
    """Host weights, packed bytes and rotating device copies, shared by the workloads that use
    the same (format, K, N): the three M values of a C5 weight need one set, not three."""

    def __init__(self, ctx):
        self.ctx = ctx
        self.host = {}
        self.sets = {}

    def host_weight(self, cfg, k, n):
        from meganeura_amd import synth

        key = (cfg, k * n)
        if key not in self.host:
            self.host[key] = synth.weights(cfg, 1, k * n).reshape(-1)
        return self.host[key].reshape(k, n)  # [K,N] and [N,K] shapes of one size share the draws

    def get(self, fmt, cfg, k, n, min_rotate_bytes):
        from meganeura_amd import capi

        dev_bytes = (k // 32) * n * (20 if fmt == Q4 else 34)
        copies = max(2, -(-min_rotate_bytes // dev_bytes)) if min_rotate_bytes else 1
        key = (fmt, cfg, k, n)
        if key not in self.sets:
            w = self.host_weight(cfg, k, n)
            self.sets[key] = (w, capi.quantize_ref(fmt, w), [])
        w, packed, devs = self.sets[key]
        while len(devs) < copies:
            devs.append(self.ctx.weight_from_packed(fmt, packed, k, n))
        return w, packed, devs[:copies]

    def drop(self, fmt, cfg, k, n):
        for wt in self.sets.pop((fmt, cfg, k, n), (None, None, []))[2]:
            wt.free()

    def free(self):
        for key in list(self.sets):
            self.drop(*key)


class Workload:
    def __init__(self, ctx, name, min_rotate_bytes, sets=None):
        from meganeura_amd import synth

        self.name = name
        fmt, m, k, n, resid, f16, cfg = WORKLOADS[name]
        self.fmt, self.m, self.k, self.n, self.resid, self.f16 = fmt, m, k, n, resid, f16
        self.ctx = ctx
        self.own_sets = sets is None
        self.sets = sets if sets is not None else WeightSets(ctx)
        self.w_host, self.packed, self.weights = self.sets.get(fmt, cfg, k, n, min_rotate_bytes)
        self.x_host = synth.activations(cfg, m, k)
        xs = self.x_host.astype(np.float16) if f16 else self.x_host
        self.a = ctx.upload(xs)
        self.c = ctx.buffer(m * n * 4)
        self.d_host = synth.activations(cfg, m, n, which=3) if resid else None
        self.d = ctx.upload(self.d_host) if resid else None
        self.bytes = algorithmic_bytes(fmt, m, k, n, resid, f16)
        self.flops = 2.0 * m * n * k
        self.is_gemm = m > 16
        self.rot = ctx.rotation(self.weights)  # built once: nothing is prepared on the host inside a timed region
        self.i = 0

    def loop(self, steps):
        """`steps` calls enqueued from C (no interpreter between the launches), weights in rotation."""
        if steps <= 0:
            return
        self.ctx.matmul_q_loop(self.a, self.rot, self.c, self.m, steps, self.d, self.f16, first=self.i)
        self.i += steps

    def preheat(self, min_ms, loop=None):
        """Launches until `min_ms` of wall clock have passed and every weight copy has been read at
        least twice: clocks are up and no copy is first touched inside a timed region."""
        loop = loop or self.loop
        t0 = time.perf_counter()
        batch = max(2 * len(self.weights), 64)
        while True:
            loop(batch)
            self.ctx.sync()
            if (time.perf_counter() - t0) * 1e3 >= min_ms:
                break

    def timed(self, steps, loop=None):
        loop = loop or self.loop
        self.ctx.sync()
        self.ctx.timer_start()
        loop(steps)
        ms = self.ctx.timer_stop()  # waits for the stop event
        return ms / steps

    def measure(self, steps, warmup, repeats, preheat_ms=100.0, loop=None):
        """Median, fastest and slowest of `repeats` timed regions of `steps` launches, in ms per step."""
        self.preheat(preheat_ms, loop)
        (loop or self.loop)(warmup)
        t = sorted(self.timed(steps, loop) for _ in range(repeats))
        return {"median": t[len(t) // 2] if len(t) % 2 else 0.5 * (t[len(t) // 2 - 1] + t[len(t) // 2]),
                "min": t[0], "max": t[-1], "repeats": repeats}

    def read_loop(self, steps, pattern=0):
        if steps > 0:
            self.ctx.weight_read_loop(self.rot, steps, first=self.i, pattern=pattern)
            self.i += steps

    def read_loop_decode_map(self, steps):
        self.read_loop(steps, pattern=1)

    def read_floor(self, steps, warmup, repeats, preheat_ms):
        """The faster of the library's two read-only passes over the same rotating copies
        (contiguous shares per workgroup; the decode kernel's own lane-to-address map), each
        pre-heated and timed like the matmul."""
        runs = {name: self.measure(steps, warmup, repeats, preheat_ms=preheat_ms, loop=loop)
                for name, loop in (("contiguous shares", self.read_loop), ("decode kernel's address map", self.read_loop_decode_map))}
        best = min(runs, key=lambda k: runs[k]["median"])
        return dict(runs[best], pattern=best, other_us={k: v["median"] * 1e3 for k, v in runs.items() if k != best})

    def output(self):
        return self.c.download(np.float32, self.m * self.n).reshape(self.m, self.n)

    def check(self):
        """The last launch's result against the oracle, within the matmul bar."""
        import oracle

        x = self.x_host.astype(np.float16).astype(np.float32) if self.f16 else self.x_host
        want = oracle.matmul_packed(self.fmt, x, oracle.quantize(self.fmt, self.w_host), self.n, self.d_host)
        oracle.assert_close(self.output(), want, 1e-3, 1e-4)
        return want

    def roofline(self, ms):
        gbs = self.bytes / (ms * 1e-3) / 1e9
        tflops = self.flops / (ms * 1e-3) / 1e12
        if self.is_gemm:
            return {"bound": "mfma", "achieved": tflops, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": tflops / MFMA_F16_PEAK_TFLOPS, "traffic": MEASURED_TRAFFIC_BYTES.get(self.name)}
        return {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": gbs / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC_BYTES.get(self.name)}

    def free(self):
        self.a.free()
        self.c.free()
        if self.d is not None:
            self.d.free()
        if self.own_sets:
            self.sets.free()


# every BASELINE workload, in the order of BASELINE.json's configs (the sweep-only entries are left out)
CONFIG_LINE = [
    "c1_q8_up_576x1536",
    "c2_q4_q_576x576", "c2_q4_kv_576x192", "c2_q4_o_576x576_add", "c2_q4_gate_up_576x3072", "c2_q4_down_1536x576_add",
    "c3_q4_lm_head_576x49152",
    "c4_q4_prefill_up_512x1024x3072", "c4_q4_prefill_down_512x3072x1024",
    "c5_q4_m1_4096x14336", "c5_q4_m4_4096x14336", "c5_q4_m16_4096x14336",
    "c5_q4_m1_14336x4096", "c5_q4_m4_14336x4096", "c5_q4_m16_14336x4096",
    "c5_q8_m1_4096x14336", "c5_q8_m4_4096x14336", "c5_q8_m16_4096x14336",
    "c5_q8_m1_14336x4096", "c5_q8_m4_14336x4096", "c5_q8_m16_14336x4096",
]


def config_table(ctx, sets, steps=200, repeats=5, preheat_ms=100.0):
    """Cache-cold time and roofline fraction of every BASELINE workload: `steps` launches per timed
    region after a pre-heat, median of `repeats`, each result checked against the oracle.  The
    pre-heat is 100 ms like the headline's: after the small workloads at the head of the table the
    first bandwidth-bound one read 9.0 instead of 7.65 us for its first 40 ms, whole regions of it,
    and 7.63 us in every measurement after (20 ms of pre-heat did not bring the clocks back up)."""
    table = {}
    last_key = None
    for name in CONFIG_LINE:
        fmt, m, k, n, resid, f16, cfg = WORKLOADS[name]
        if last_key is not None and last_key != (fmt, cfg, k, n):
            sets.drop(*last_key)  # the rotating copies of the previous weight are no longer needed
        last_key = (fmt, cfg, k, n)
        wl = Workload(ctx, name, 512 << 20, sets)
        r = wl.measure(steps, 20, repeats, preheat_ms)
        wl.check()
        roof = wl.roofline(r["median"])
        table[name] = {"us": r["median"] * 1e3, "us_min": r["min"] * 1e3, "us_max": r["max"] * 1e3,
                       # read right behind the timed regions: one idle wave, and under a matrix-instruction load
                       "engine_mhz": round(ctx.engine_clock_mhz()), **dict(zip(("engine_mhz_loaded", "load_cycles_per_round"), map(round, ctx.engine_probe()))),
                       "bound": roof["bound"], "achieved": roof["achieved"], "unit": roof["unit"], "frac": roof["frac"],
                       "algorithmic_bytes": wl.bytes}
        if m == 1 and wl.bytes >= (8 << 20):
            # a bandwidth-bound one-row call beside its own floor on this box: the faster of the two
            # read-only passes over the same rotating copies, pre-heated and timed the same way
            fl = wl.read_floor(steps, 20, repeats, preheat_ms)
            table[name]["read_floor_us"] = fl["median"] * 1e3
            table[name]["frac_of_read_floor"] = fl["median"] / r["median"]
        if m > 4 and not f16:
            # f32 activations at M >= 5: the figure above is the context's default (activations of any
            # magnitude, the rescaling kernels); beside it, the same call on a context that was promised
            # activations in the fp16 range (mgn_ctx_set_activation_range), where the plans differ
            from meganeura_amd import capi
            if capi.matmul_plan(fmt, m, k, n).route != capi.matmul_plan(fmt, m, k, n, fp16_range=True).route:
                ctx.set_activation_range(True)
                try:
                    rp = wl.measure(steps, 20, repeats, preheat_ms)
                    wl.check()
                finally:
                    ctx.set_activation_range(False)
                table[name]["us_fp16_range"] = rp["median"] * 1e3
                table[name]["frac_fp16_range"] = wl.roofline(rp["median"])["frac"]
        wl.free()
    if last_key is not None:
        sets.drop(*last_key)
    return table


def ffn_chain_times(ctx, steps=200, repeats=5, hidden=4096, inter=14336):
    """The Llama-3-8B-shaped FFN at one token as the dependent pair it is: rms_norm -> gate | up
    (4096 x 28672) and SwiGLU -> down + residual (14336 x 4096), 110.1 MB of Q4 weights, two launches
    (each with its neighbour folded in), weights rotating through >= 512 MiB of copies.  Beside it the
    same pair as ONE chain launch (mgn_chain_*), which is not what the library's Session would do
    with weights of this size: the chain's looped stage streams them more slowly."""
    import oracle
    from meganeura_amd import capi, synth

    x = synth.activations(5, 1, hidden, which=77)
    g = (1.0 + synth.normal(78, hidden, 0.1)).astype(np.float32)
    wgu, wd = synth.weights(5, hidden, 2 * inter, which=79), synth.weights(5, inter, hidden, which=80)
    first = (ctx.weight(Q4, wgu), ctx.weight(Q4, wd))
    packed = (first[0].export_ref(), first[1].export_ref())
    nbytes = packed[0].size + packed[1].size
    copies = max(2, (512 << 20) // nbytes + 1)
    pairs = [first] + [(ctx.weight_from_packed(Q4, packed[0], hidden, 2 * inter), ctx.weight_from_packed(Q4, packed[1], inter, hidden))
                       for _ in range(copies - 1)]
    bx, bg = ctx.upload(x), ctx.upload(g)
    bgu, by = ctx.buffer(2 * inter * 4), ctx.buffer(hidden * 4)

    def separate(n, at):
        for i in range(n):
            wa, wb = pairs[(at + i) % copies]
            ctx.matmul_q_rms_norm(bx, bg, 1e-5, wa, bgu, 1)
            ctx.matmul_q_swiglu(bgu, wb, by, 1, bx)

    chains = [ctx.chain([dict(w=wa, a=bx, c=bgu, prologue=capi.PROLOGUE_RMS_NORM, norm_weight=bg, eps=1e-5),
                         dict(w=wb, a=bgu, c=by, prologue=capi.PROLOGUE_SWIGLU, d=bx)]) for wa, wb in pairs]

    def chained(n, at):
        for i in range(n):
            chains[(at + i) % copies].run()

    # the result against numpy pointwise operations + the oracle's matmul (on the first copy)
    deq = lambda w: oracle.dequantize(Q4, oracle.quantize(Q4, w), *w.shape)
    x64 = x.astype(np.float64)
    n1 = (x64 / np.sqrt((x64 ** 2).mean() + 1e-5) * g).astype(np.float32)
    gu = oracle.matmul_f32(n1, deq(wgu))
    gg, uu = gu[:, :inter].astype(np.float64), gu[:, inter:].astype(np.float64)
    want = oracle.matmul_f32((gg / (1.0 + np.exp(-gg)) * uu).astype(np.float32), deq(wd), x)
    res = {}
    for name, fn in (("separate", separate), ("chain", chained)):
        fn(1, 0)
        oracle.assert_close(by.download(np.float32, hidden).reshape(1, -1), want, 1e-3, 1e-4)
        fn(600, 0)
        ctx.sync()
        t = []
        for r in range(repeats):
            ctx.timer_start()
            fn(steps, r * 3)
            t.append(ctx.timer_stop() / steps)
        res[name] = sorted(t)[len(t) // 2] * 1e3
    bytes_ = nbytes // 20 * 20 + 4 * (hidden + 2 * inter) * 2 + 4 * hidden * 3  # weights + activations in and out of both matmuls + residual
    for c in chains:
        c.free()
    for h in [bx, bg, bgu, by] + [w for p in pairs for w in p]:
        h.free()
    return {"us": res["separate"], "chain_us": res["chain"], "algorithmic_bytes": bytes_, "bound": "hbm",
            "achieved": bytes_ / (res["separate"] * 1e-6) / 1e9, "unit": "GB/s",
            "frac": bytes_ / (res["separate"] * 1e-6) / 1e9 / HBM_PEAK_GBS,
            "what": "rms_norm -> gate|up (4096 x 28672) then SwiGLU -> down + residual (14336 x 4096), Q4, one token: two launches, "
                    "cache-cold; chain_us = the same pair as one chain launch"}


def decode_layer_times(steps, warmup, layers=8):
    """C2 as the reference runs it: SmolLM2-135M decode layers' matmuls through the
    Graph/Session surface (models/smollm2.rs:340-414 without the attention core): rms_norm,
    q/k/v, o-projection + residual, rms_norm, gate||up as one fused matmul, SwiGLU, down +
    residual -- 9 dispatches per layer after the optimizer's fusions, `layers` of them chained
    in one session so that the per-step cost of the host loop is spread as in a real model.
    Returns microseconds per layer: every dispatch its own launch, norms and SwiGLU folded
    into the matmuls (the default), and the folded step replayed as one captured graph."""
    from meganeura_amd import capi, synth
    from meganeura_amd.graph import Graph, build_inference_session

    hidden, kv, inter = 576, 192, 1536
    g = Graph()
    x = g.input("x", [1, hidden])
    attn = g.input("attn", [1, hidden])
    outs, shapes = [], {}
    for l in range(layers):
        n1 = g.rms_norm(x, g.parameter(f"norm1.{l}", [hidden]), 1e-5)
        q = g.matmul(n1, g.parameter_q4(f"wq.{l}", [hidden, hidden]))
        k = g.matmul(n1, g.parameter_q4(f"wk.{l}", [hidden, kv]))
        v = g.matmul(n1, g.parameter_q4(f"wv.{l}", [hidden, kv]))
        h = g.add(g.matmul(attn, g.parameter_q4(f"wo.{l}", [hidden, hidden])), x)
        n2 = g.rms_norm(h, g.parameter(f"norm2.{l}", [hidden]), 1e-5)
        gate = g.matmul(n2, g.parameter_q4(f"wg.{l}", [hidden, inter]))
        up = g.matmul(n2, g.parameter_q4(f"wu.{l}", [hidden, inter]))
        x = g.add(g.matmul(g.swiglu(gate, up), g.parameter_q4(f"wd.{l}", [inter, hidden])), h)
        outs += [q, k, v]
        shapes.update({f"wq.{l}": (hidden, hidden), f"wk.{l}": (hidden, kv), f"wv.{l}": (hidden, kv),
                       f"wo.{l}": (hidden, hidden), f"wg.{l}": (hidden, inter), f"wu.{l}": (hidden, inter),
                       f"wd.{l}": (inter, hidden)})
    g.set_outputs([x] + outs)
    sess = build_inference_session(g)
    for i, (name, (kk, nn)) in enumerate(shapes.items()):
        sess.set_parameter(name, synth.weights(2, kk, nn, which=i % 7))
    for l in range(layers):
        sess.set_parameter(f"norm1.{l}", np.ones(hidden, np.float32))
        sess.set_parameter(f"norm2.{l}", np.ones(hidden, np.float32))
    sess.set_input("x", synth.activations(2, 1, hidden, which=0))
    sess.set_input("attn", synth.activations(2, 1, hidden, which=1))
    ctx = sess.context()
    res = {"layers": layers, "dispatches_per_layer": len(sess.plan()) // layers}
    for label, fusion, replay, chains in (("unfused", False, False, False), ("fused", True, False, False),
                                          ("fused_graph", True, True, False), ("chain", True, False, True)):
        sess.set_fusion(fusion)
        sess.set_graph_replay(replay)
        sess.set_chains(chains)
        res[label + "_launches_per_layer"] = sess.num_launches() / layers
        for _ in range(warmup + 2):
            sess.step()
        ctx.sync()
        ctx.timer_start()
        for _ in range(steps):
            sess.step()
        ms = ctx.timer_stop()
        ctx.sync()
        res[label + "_us_per_layer"] = ms * 1e3 / steps / layers
    sess.close()
    return res


def quantizer_times(ctx, fmt=Q4, k=4096, n=14336):
    """set_parameter's cost for one C5 weight (58.7 M elements): the host quantizer of the
    library (threads over block rows; the reference's is a single-threaded scalar loop,
    src/runtime.rs:2035-2102) and the bit-identical device kernel fed from a device buffer."""
    from meganeura_amd import capi, synth

    w = synth.weights(5, k, n)
    t0 = time.perf_counter()
    packed = capi.quantize_ref(fmt, w)
    host_s = time.perf_counter() - t0
    src = ctx.upload(w)
    wt = ctx.weight_from_device(fmt, src, k, n)  # warm-up: allocation paths, kernel load
    wt.free()
    ctx.sync()
    ctx.timer_start()
    wt = ctx.weight_from_device(fmt, src, k, n)
    dev_ms = ctx.timer_stop()
    same = bool((wt.export_ref() == packed).all())
    wt.free()
    src.free()
    return {"workload": f"quantize_{'q4' if fmt == Q4 else 'q8'}_{k}x{n}", "host_ms": host_s * 1e3,
            "host_GBs_f32_in": w.nbytes / host_s / 1e9, "device_ms": dev_ms,
            "device_GBs_f32_in": w.nbytes / (dev_ms * 1e-3) / 1e9, "device_bytes_equal_host": same}


def copy_ceiling(ctx, nbytes=256 << 20, reps=20):
    """What a plain device-to-device copy moves on this box (bytes read + bytes written per
    second): an achievable figure to set beside the published HBM peak."""
    src, dst = ctx.buffer(nbytes), ctx.buffer(nbytes)
    for _ in range(3):
        ctx.copy(dst, src, nbytes)
    ctx.sync()
    ctx.timer_start()
    for _ in range(reps):
        ctx.copy(dst, src, nbytes)
    ms = ctx.timer_stop() / reps
    ctx.sync()
    src.free()
    dst.free()
    return 2.0 * nbytes / (ms * 1e-3) / 1e9


def cpu_baseline(wl, cpu_seconds=20.0):
    """The reference's tiled dequant-on-load algorithm restated for the CPU
    (oracle/mgn_oracle.c: orc_matmul_q_tiled), one OpenMP task per workgroup, on
    this box's host cores.  Checker infrastructure used as the timing baseline
    only; it is never part of the product path."""
    import oracle

    x = wl.x_host.astype(np.float16).astype(np.float32) if wl.f16 else wl.x_host
    packed_ref = oracle.quantize(wl.fmt, wl.w_host)
    t0 = time.perf_counter()
    out = oracle.matmul_packed(wl.fmt, x, packed_ref, wl.n, wl.d_host, tiled=True)
    first = time.perf_counter() - t0
    # sample size: about `cpu_seconds` of CPU work (threads x wall clock), never fewer than 2 calls
    reps = int(max(1, min(500, cpu_seconds / oracle.num_threads() / max(first, 1e-4) - 1)))
    t0 = time.perf_counter()
    for _ in range(reps):
        oracle.matmul_packed(wl.fmt, x, packed_ref, wl.n, wl.d_host, tiled=True)
    per = (time.perf_counter() - t0) / reps
    return out, {
        "value": wl.bytes / per / 1e9,
        "unit": "GB/s",
        "cores": oracle.num_threads(),
        "kind": "port",
        "ms_per_call": per * 1e3,
        "sample": f"{reps + 1} full calls of {wl.name}, about {(reps + 1) * per * oracle.num_threads():.0f} s of CPU work "
                  "(64x64x32-tiled per-element dequant, the reference shader's algorithm, OpenMP over workgroups)",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--repeats", type=int, default=0,
                    help="timed regions of --steps launches each (median reported); default: at least 5, "
                         "more when --steps is small, so that about 2000 launches are timed in all")
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS))
    ap.add_argument("--sweep", action="store_true", help="also measure cache-warm figures and the quantizers (stderr)")
    ap.add_argument("--sweep-out", default=None, help="with --sweep: also write the table to this JSON file")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-configs", action="store_true", help="skip the per-configuration table of the JSON line")
    ap.add_argument("--profile", action="store_true",
                    help="for rocprofv3 runs: only the timed cache-cold workload plus one 256 MiB device copy "
                         "(a known size to calibrate FETCH_SIZE / WRITE_SIZE against); no CPU leg, no warm leg")
    ap.add_argument("--profile-chains", action="store_true",
                    help="for rocprofv3 runs: only the decode layer through the Session (8 layers a step, as one chain "
                         "launch a layer and as separate launches) and the FFN pair, then exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU part (column-parallel "
                 "sharding needs no exchange); run with --gpus 1")
    if args.steps <= 0:
        sys.exit("--steps must be positive")
    repeats = args.repeats if args.repeats > 0 else max(5, min(100, -(-2000 // args.steps)))

    from meganeura_amd import capi
    import oracle

    if args.profile_chains:
        ctx = capi.Context(0)
        out = {"c5_q4_ffn_m1": ffn_chain_times(ctx), "c2_q4_decode_layer_session": decode_layer_times(200, 20)}
        ctx.close()
        print(json.dumps(out))
        return

    ctx = capi.Context(0)
    sets = WeightSets(ctx)
    wl = Workload(ctx, args.workload, 512 << 20, sets)
    timing = wl.measure(args.steps, args.warmup, repeats, preheat_ms=20.0 if args.profile else 100.0)
    engine_mhz = round(ctx.engine_clock_mhz())
    engine_mhz_loaded, load_cycles_per_round = map(round, ctx.engine_probe())
    ms = timing["median"]
    want = wl.check()  # the timed kernel's result against the oracle, before anything is reported

    floor = None if args.profile else wl.read_floor(args.steps, args.warmup, repeats, preheat_ms=100.0)

    gbs = wl.bytes / (ms * 1e-3) / 1e9
    tflops = wl.flops / (ms * 1e-3) / 1e12

    if args.profile:
        args.no_cpu = args.no_configs = True
        cal = 256 << 20
        src, dst = ctx.buffer(cal), ctx.buffer(cal)
        ctx.copy(dst, src, cal)
        ctx.sync()
        src.free()
        dst.free()

    cpu = None
    if not args.no_cpu:
        cpu_out, cpu = cpu_baseline(wl)
        oracle.assert_close(cpu_out, want, 1e-3, 1e-4)

    # cache-warm figure for the same shape (one weight, reused every step)
    warm = copy_gbs = None
    if not args.profile:
        ww = Workload(ctx, args.workload, 0, sets)
        warm = ww.measure(args.steps, args.warmup, repeats, preheat_ms=20.0)
        ww.free()
        copy_gbs = copy_ceiling(ctx)

    line = {
        "metric": "Q4/Q8 GEMV HBM GB/s (% of peak) + us/call; prefill dequant-GEMM TFLOP/s",
        "value": tflops if wl.is_gemm else gbs,
        "unit": "TFLOP/s" if wl.is_gemm else "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "us_per_call": ms * 1e3,
        "repeats": repeats,
        "us_per_call_min": timing["min"] * 1e3,
        "us_per_call_max": timing["max"] * 1e3,
        "engine_mhz": engine_mhz,
        "engine_mhz_loaded": engine_mhz_loaded,
        "load_cycles_per_round": load_cycles_per_round,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": args.workload,
            "format": "q4" if wl.fmt == Q4 else "q8",
            "m": wl.m, "k": wl.k, "n": wl.n,
            "algorithmic_bytes": wl.bytes,
            "cache": f"cold: rotating {len(wl.weights)} weight copies",
            "timing": f"median of {repeats} timed regions of {args.steps} back-to-back launches, after a pre-heat of "
                      ">= 100 ms of launches over every copy and the warm-up steps",
        },
        "roofline": wl.roofline(ms),
        "cpu_baseline": cpu,
        "cache_warm": None if warm is None else
        {"us_per_call": warm["median"] * 1e3, "GB/s": wl.bytes / (warm["median"] * 1e-3) / 1e9},
        "pct_of_hbm_peak": 100.0 * gbs / HBM_PEAK_GBS,
        "copy_ceiling": None if copy_gbs is None else
        {"GB/s": copy_gbs, "what": "256 MiB device-to-device copy, bytes read + written per second",
         "pct_of_it": 100.0 * gbs / copy_gbs},
        "read_floor": None if floor is None else
        {"us_per_launch": floor["median"] * 1e3, "GB/s": wl.bytes / (floor["median"] * 1e-3) / 1e9,
         "what": "the faster of two kernels that only read the same rotating weight copies (quants and scales), pre-heated "
                 "and timed the same way: one launch plus one pass over the packed bytes on this box",
         "pattern": floor["pattern"], "other_pattern_us": floor["other_us"],
         "pct_of_it": 100.0 * floor["median"] / ms},
    }
    wl.free()

    if not args.no_configs:
        line["configs"] = config_table(ctx, sets)
        line["configs"]["c5_q4_ffn_m1"] = ffn_chain_times(ctx)
        layer = decode_layer_times(200, 20)
        line["configs"]["c2_q4_decode_layer_session"] = {
            "us": layer["chain_us_per_layer"],  # the session's default: the whole step's matmuls as one chain launch
            "launches": layer["chain_launches_per_layer"],
            "separate_launches_us": layer["fused_us_per_layer"], "separate_launches": layer["fused_launches_per_layer"],
            "unfused_us": layer["unfused_us_per_layer"],
            "graph_replay_us": layer["fused_graph_us_per_layer"],  # the separate launches captured once and replayed
            "dispatches": layer["dispatches_per_layer"],
            "what": "one SmolLM2-135M decode layer's matmuls, norms and SwiGLU through the Graph/Session surface, per layer "
                    "(8 layers chained in one session)"}

    if args.sweep:
        rows = []
        for name in WORKLOADS:
            row = {"workload": name}
            for label, rot in (("cold", 512 << 20), ("warm", 0)):
                w = Workload(ctx, name, rot, sets)
                r = w.measure(200, 20, 5, preheat_ms=100.0)
                t = r["median"]
                row[label + "_us"] = t * 1e3
                row[label + "_GBs"] = w.bytes / (t * 1e-3) / 1e9
                row[label + "_TFLOPs"] = w.flops / (t * 1e-3) / 1e12
                row["bytes"] = w.bytes
                if rot:  # the read-only pass over the same rotating copies, see read_floor above
                    row["read_floor_us"] = w.read_floor(200, 20, 5, preheat_ms=5.0)["median"] * 1e3
                w.free()
            fmt, m, k, n, resid, f16, cfg = WORKLOADS[name]
            sets.drop(fmt, cfg, k, n)
            row["cold_pct_hbm"] = 100.0 * row["cold_GBs"] / HBM_PEAK_GBS
            rows.append(row)
            print(json.dumps(row), file=sys.stderr, flush=True)
        layer = {"workload": "c2_q4_decode_layer_session", **decode_layer_times(200, 20)}
        rows.append(layer)
        print(json.dumps(layer), file=sys.stderr, flush=True)
        for fmt in (Q4, Q8):
            row = quantizer_times(ctx, fmt)
            rows.append(row)
            print(json.dumps(row), file=sys.stderr, flush=True)
        if args.sweep_out:
            with open(args.sweep_out, "w") as f:
                json.dump(rows, f, indent=1)

    sets.free()
    ctx.close()
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
