#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  Headline (`value`): W8A8 prefill GEMM throughput, in TOP/s, over the
seven projections of one Llama-3-8B layer at M = 2048 tokens (q, k, v, o, gate, up, down;
893 353 197 568 integer ops per step), run as models::llama runs them: q|k|v and gate|up as fused
products over one input (four calls, each = per-row activation quantisation + i8 MFMA GEMM +
f32 rescale), inputs resident in HBM: two sets of layer weights (436 MB, more than the Infinity
Cache) are used alternately, and the step runs untimed for 0.2 s before the W warm-up steps so
that clocks and caches have settled.
The same line carries the decode leg of the metric (`decode_gemv`: M = 1 int8 GEMV GB/s at
the 8B FFN shapes, weights rotated through more distinct buffers than the 256 MB Infinity
Cache holds), the Q4_0 decode GEMV (`gguf_q4_0_gemv`), a `roofline` object per dominant
kernel (durations from HIP events recorded by the library on its own stream) and the CPU
baseline (`cpu_baseline`: the scalar oracle on this host's cores, one thread, bounded sample;
cfg1, cfg2 and cfg4 carry their own full-size `cpu_baseline`).

Every section reports `ms_per_step` (K timed steps between two events, as the contract asks) and,
from a second pass with an event after every step, the median / min / std of the single steps
(the reference's protocol, benches/wallclock.rs:19-41).  Inputs come from the reference's own
generators restated in peregrine_amd/synth.py (Philox 4x32-10 / Xoshiro256++ with Box-Muller,
src/random.rs), run as torch array code on the device.  `ceilings` holds what the part delivered in
this very run on three probes (register-only int8 MFMA loop, pure HBM read stream, the shader
clock inside a GEMM tile); roofline fractions stay against the published peaks.

torch is used for device memory, input synthesis and the whole-step timing events only.
"""
import argparse
import ctypes as C
import json
import os
import statistics
import subprocess
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "W8A8 GEMM TOPS (%int8 MFMA peak) + M=1 decode GEMV GB/s (%HBM), 8B shapes"
PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, published
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, published
M_PREFILL = 2048
# (name, K, N) of one Llama-3-8B layer: d 4096, 8 KV heads (kv dim 1024), ffn 14336
LAYER = [("q_proj", 4096, 4096), ("k_proj", 4096, 1024), ("v_proj", 4096, 1024), ("o_proj", 4096, 4096),
         ("gate_proj", 4096, 14336), ("up_proj", 4096, 14336), ("down_proj", 14336, 4096)]
LAYER_OPS = sum(2 * M_PREFILL * k * n for _, k, n in LAYER)  # 893 353 197 568
SETTLE_S = 0.2  # untimed run of the headline step before its warm-up, seconds


def load_traffic():
    """profiles/hbm_traffic.json: HBM bytes per launch, per kernel family and launch size
    (work-items), derived from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this benchmark and
    scaled by a plain copy of known size (the file names the commands).  Absent file -> traffic is
    reported as null."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            return json.load(f).get("bytes_per_launch_by_size", {})
    except (OSError, ValueError):
        return {}


TRAFFIC = load_traffic()
LAUNCHES_SEEN = {}  # kernel family -> launch sizes (work-items) of this run, reported as `launch_work_items`


def gemv_bytes(k, n):
    """Algorithmic bytes of one M = 1 W8A8 product: i8 weights + w scales + f32 x + f32 out."""
    return k * n + 4 * n + 4 * k + 4 * n


class Bench:
    """The device, the library context and the helpers every section uses."""

    def __init__(self, args):
        import torch
        from peregrine_amd import _ffi, Context, synth

        if not torch.cuda.is_available():
            sys.exit("bench.py: no GPU visible; peregrine_amd has no CPU path to measure")
        self.args, self.torch, self.synth, self.ffi = args, torch, synth, _ffi
        self.dev = torch.device("cuda:0")
        torch.cuda.set_device(self.dev)
        # A dedicated (non-null) stream shared by torch and the library, so the torch events
        # that bracket the timed region see the library's kernels.
        self.stream = torch.cuda.Stream(device=self.dev)
        torch.cuda.set_stream(self.stream)
        assert self.stream.cuda_stream != 0
        self.ctx = Context(0, stream=self.stream.cuda_stream)
        assert self.ctx.stream == self.stream.cuda_stream
        self.lib, self.check = _ffi.lib, _ffi.check
        self.h = self.ctx.handle
        self.cpu = not args.skip_cpu
        self.orc = load_oracle() if self.cpu else None
        self.i = 0  # rotation counter of the sections that cycle through several weight buffers
        self.dsteps = max(args.steps * 10, 100)

    @staticmethod
    def ptr(t):
        return C.c_void_p(t.data_ptr())

    def normal(self, seed, shape, std=1.0):
        """N(0, std) as the reference's random::normal would fill a tensor of that size after
        random::seed(seed) (Philox path from 200 000 elements, Xoshiro below), on the device."""
        n = 1
        for d in shape:
            n *= d
        return self.synth.Random(seed).normal(n, 0.0, std, device=self.dev).reshape(shape).contiguous()

    def make_weight(self, k, n, seed, keep=None):
        """[k, n] ~ N(0, 0.02) quantised on the device; `keep` collects the f32 matrix on the host."""
        w = self.normal(seed, (k, n), 0.02)
        h = C.c_void_p()
        self.check(self.lib.pg_qtensor_from_f32_dev(self.h, self.ptr(w), k, n, C.byref(h)))
        if keep is not None:
            keep.append(w.cpu().numpy())
        del w
        return h

    def make_acts(self, m, k, seed):
        """N(0,1) rows with 1 % of the channels (a fixed set from the sequential stream) x20."""
        a = self.normal(seed, (m, k))
        chan = self.synth.Random(seed + 1).distinct_below(max(1, k // 100), k)
        a[:, self.torch.tensor(chan, device=self.dev)] *= 20.0
        return a.contiguous()

    def timed(self, fn, steps, warmup):
        """W untimed steps, then K steps between two events (-> ms_per_step), then K more with an
        event after each (-> median / min / std of single steps)."""
        torch = self.torch
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(self.stream)
        for _ in range(steps):
            fn()
        e1.record(self.stream)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        evs[0].record(self.stream)
        for i in range(steps):
            fn()
            evs[i + 1].record(self.stream)
        torch.cuda.synchronize()
        per = [evs[i].elapsed_time(evs[i + 1]) for i in range(steps)]
        return {"ms_per_step": ms, "median_ms": statistics.median(per), "min_ms": min(per),
                "std_ms": statistics.pstdev(per) if len(per) > 1 else 0.0}

    @staticmethod
    def stats(t, digits=5):
        return {k: round(t[k], digits) for k in ("ms_per_step", "median_ms", "min_ms", "std_ms")}

    def profiled(self, fn, steps):
        """Per-kernel durations from the library's HIP events: each dispatch carries a start
        and a stop event stamped with the kernel's own begin/end on the stream it runs on
        (hipExtLaunchKernel), so the figures are comparable with a rocprofv3 kernel trace.
        Returns ({name: (avg_ms, launches)}, {name: {work-items of a launch: launches}})."""
        self.ctx.profile_begin()
        for _ in range(steps):
            fn()
        tot = {name: (total / n, n) for name, (total, n) in self.ctx.profile_end().items()}
        return tot, self.ctx.profile_grids()

    @staticmethod
    def traffic_for(kernel, grids):
        """HBM bytes per launch of a kernel family: the committed rocprofv3 --pmc figures per launch
        size, weighted by the launches this run made of each size -- but only while those sizes are
        exactly the ones the counters were taken on; otherwise None (the kernel or its dispatch
        changed since: the summary is stale)."""
        got = grids.get(kernel, {})
        LAUNCHES_SEEN[kernel] = sorted(got)
        have = TRAFFIC.get(kernel)
        if not have or sorted(int(g) for g in have) != sorted(got):
            return None
        return int(sum(n * have[str(g)] for g, n in got.items()) / sum(got.values()))

    def ceilings(self):
        """What the part delivers on three probes, measured now (fractions stay against the published peaks)."""
        tops, ghz, gbs, g_ghz, loop_us = (C.c_double() for _ in range(5))
        self.check(self.lib.pg_probe_mfma_i8(self.h, 20000, C.byref(tops), C.byref(ghz)))
        self.check(self.lib.pg_probe_hbm_read(self.h, 256 << 20, 3, 30, C.byref(gbs)))
        self.check(self.lib.pg_probe_gemm_clock(self.h, 2048, 4096, 14336, C.byref(g_ghz), C.byref(loop_us)))
        # a pure read of one launch's bytes, best of a few launch shapes (workgroups, threads, loads in flight):
        # what a one-row product of that size could reach if it did nothing but read
        small = {}
        shapes = ((4096, 256, 4), (2048, 512, 4), (2048, 256, 8), (1024, 512, 8), (1024, 256, 16), (512, 1024, 4))
        for label, nbytes, bufs in (("33MB", 33103872, 10), ("59MB", 58851328, 6), ("118MB", 117702656, 4)):
            best = (0.0, None)   # cfg4's largest launch, cfg2's down, cfg2's gate|up
            for wgs, thr, inflight in shapes:
                g = C.c_double()
                self.check(self.lib.pg_probe_hbm_read_shaped(self.h, nbytes, bufs, 200, wgs, thr, inflight, C.byref(g)))
                if g.value > best[0]:
                    best = (g.value, (wgs, thr, inflight))
            small[label] = {"gbs": round(best[0], 1), "us": round(nbytes / best[0] / 1e3, 2),
                            "workgroups_threads_loads_in_flight": list(best[1])}
        return {"hbm_read_stream_per_launch_size": small, "int8_mfma_registers_only_tops": round(tops.value, 1), "its_shader_clock_ghz": round(ghz.value, 3),
                "hbm_read_stream_gbs": round(gbs.value, 1), "gemm_tile_shader_clock_ghz": round(g_ghz.value, 3),
                "gemm_tile_k_loop_us": round(loop_us.value, 2),
                "int8_peak_at_gemm_clock_tops": round(256 * 8192 * g_ghz.value / 1e3, 1),
                "note": "measured in this run by pg_probe_*: 8 wavefronts per CU issuing only v_mfma_i32_32x32x32_i8 on "
                        "pseudo-random registers; 128-bit non-temporal reads over 3 x 256 MiB; shader cycles / wall clock "
                        "inside the K loop of the 256x256 tile of a [2048x4096]x[4096x14336] product"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU baseline legs")
    ap.add_argument("--only-headline", action="store_true", help="cfg3 (and the ceilings) only")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain 512 MiB device copies (counter calibration under rocprofv3 --pmc)")
    ap.add_argument("--probe-shapes", action="store_true",
                    help="instead of the benchmark: the pure read probe over launch shapes (workgroups x threads x loads in "
                         "flight) at the byte counts of the one-row products, one JSON line")
    ap.add_argument("--cache-residency", action="store_true",
                    help="instead of the benchmark: the one-row products timed with 1 .. 12 tensors rotated "
                         "(weights served by the L2s, the Infinity Cache, HBM), one JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; every kernel here runs at its real "
                 "single-GPU shape. Run with --gpus 1.")

    import numpy as np

    B = Bench(args)
    torch, lib, check, ptr, dev = B.torch, B.lib, B.check, B.ptr, B.dev
    if args.probe_shapes:
        print(json.dumps(probe_shapes(B)), flush=True)
        return
    if args.cache_residency:
        print(json.dumps(cache_residency(B)), flush=True)
        return

    # ------------------------------------------------------------------ prefill (headline)
    # Two layers' worth of weights (436 MB), used alternately: more than the 256 MB Infinity Cache
    # holds, so every step streams its weights from HBM as a model with many layers would
    # (with one set reused every step the layer runs about 3 % faster).
    weight_sets = []
    for s_i in range(2):
        ws = {}
        for j, (name, k, n) in enumerate(LAYER):
            ws[name] = B.make_weight(k, n, 5678 + 16 * s_i + j)
        weight_sets.append(ws)
    weights = weight_sets[0]
    acts = {4096: B.make_acts(M_PREFILL, 4096, 1234), 14336: B.make_acts(M_PREFILL, 14336, 1236)}
    outs = {n: torch.empty(M_PREFILL, n, device=dev, dtype=torch.float32) for n in (4096, 1024, 14336)}
    # The layer as models::llama runs it: q|k|v and gate|up are fused products over one input
    # (src/models/llama/attention.rs:51-71,84; decoder.rs:49-67,78), so the step is four calls:
    # each quantises its activation rows once; the multi-weight calls are one launch each.
    outs["k"], outs["v"] = (torch.empty(M_PREFILL, 1024, device=dev, dtype=torch.float32) for _ in range(2))
    outs["up"] = torch.empty(M_PREFILL, 14336, device=dev, dtype=torch.float32)
    VP3, VP2 = C.c_void_p * 3, C.c_void_p * 2
    qkv_out = VP3(outs[4096].data_ptr(), outs["k"].data_ptr(), outs["v"].data_ptr())
    gu_out = VP2(outs[14336].data_ptr(), outs["up"].data_ptr())
    for ws in weight_sets:
        ws["qkv_tab"] = VP3(ws["q_proj"].value, ws["k_proj"].value, ws["v_proj"].value)
        ws["gu_tab"] = VP2(ws["gate_proj"].value, ws["up_proj"].value)

    def prefill_step():
        ws = weight_sets[B.i % len(weight_sets)]
        B.i += 1
        a4, a14 = ptr(acts[4096]), ptr(acts[14336])
        check(lib.pg_matmul_quantized_multi_dev(B.h, a4, M_PREFILL, 4096, ws["qkv_tab"], 3, qkv_out))
        check(lib.pg_matmul_quantized_dev(B.h, a4, M_PREFILL, 4096, ws["o_proj"], ptr(outs[4096]), None))
        check(lib.pg_matmul_quantized_multi_dev(B.h, a4, M_PREFILL, 4096, ws["gu_tab"], 2, gu_out))
        check(lib.pg_matmul_quantized_dev(B.h, a14, M_PREFILL, 14336, ws["down_proj"], ptr(outs[4096]), None))

    # Clocks and caches need tens of milliseconds of this work to settle (a 3 ms warm-up leaves
    # the layer about 8 % slower than its steady state): run it untimed for SETTLE_S first, then
    # the W warm-up steps and the K timed ones as asked.
    t_settle = time.time()
    while time.time() - t_settle < SETTLE_S:
        for _ in range(10):
            prefill_step()
        torch.cuda.synchronize()
    t_head = B.timed(prefill_step, args.steps, args.warmup)
    ms_step = t_head["ms_per_step"]
    tops = LAYER_OPS / (ms_step * 1e-3) / 1e12
    prof, grids = B.profiled(prefill_step, args.steps)
    gemm_avg_ms, g_n = prof["gemm_w8a8"]
    q_avg_ms, q_n = prof["quantize_rows"]
    gemm_lps = g_n / args.steps  # GEMM launches per step
    gemm_tops = (LAYER_OPS / gemm_lps) / (gemm_avg_ms * 1e-3) / 1e12
    quant_ks = (4096, 4096, 4096, 14336)  # one quantisation per call of the step
    quant_bytes = sum(M_PREFILL * k * 4 + M_PREFILL * k + M_PREFILL * 4 for k in quant_ks)
    roofline = {"kernel": "gemm_w8a8_kernel (i8 MFMA 32x32x32; the 7 products as 5 launches: q|k|v, o, gate, up, down)", "bound": "mfma",
                "achieved": round(gemm_tops, 1), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                "frac": round(gemm_tops / PEAK_INT8_TOPS, 4), "traffic": B.traffic_for("gemm_w8a8", grids),
                "ops_per_launch": int(LAYER_OPS / gemm_lps), "launches_per_step": gemm_lps, "avg_launch_ms": round(gemm_avg_ms, 4),
                "note": "an int8 multiply-add counts as 2 ops; duration from the HIP events attached to each dispatch"}
    act_quant = {"kernel": "quantize_rows_vec4_kernel", "bound": "hbm",
                 "achieved": round(quant_bytes / len(quant_ks) / (q_avg_ms * 1e-3) / 1e9, 1),
                 "peak": PEAK_HBM_GBS, "unit": "GB/s", "avg_launch_ms": round(q_avg_ms, 4),
                 "traffic": B.traffic_for("quantize_rows", grids)}
    act_quant["frac"] = round(act_quant["achieved"] / PEAK_HBM_GBS, 4)
    ceil = None if args.calibrate_copy else B.ceilings()  # (counter runs measure traffic only)
    if ceil:  # the same achieved rate against what the part's matrix cores sustained in this run on operands in registers
        roofline["frac_of_measured_ceiling"] = round(gemm_tops / ceil["int8_mfma_registers_only_tops"], 4)

    # Per product shape: this library's GEMM kernel beside the vendor library's int8 GEMM
    # (torch._int_mm = hipBLASLt; same operand layouts, i32 output without the rescale) on
    # random int8 operands.  Both run for 50 ms first (clocks settle under the same load).
    # `gemm_w8a8_ms` is kernel time from the dispatch events; `gemm_w8a8_stream_event_ms` and the
    # vendor's figures are on one clock: the mean of single calls between stream events (launch gap
    # included), ours less the kernel time of its quantisation launch.  A
    # calibration of what int8 matrix-core code reaches on this part at these sizes, not a figure
    # of this library.
    def settle(fn, seconds=0.05):
        t0 = time.time()
        while time.time() - t0 < seconds:
            for _ in range(20):
                fn()
            torch.cuda.synchronize()

    vendor = []
    for name, k, n in (() if args.calibrate_copy else (("q/o_proj", 4096, 4096), ("gate/up_proj", 4096, 14336), ("down_proj", 14336, 4096))):
        wname = {"q/o_proj": "q_proj", "gate/up_proj": "gate_proj", "down_proj": "down_proj"}[name]

        def one_product():
            ws = weight_sets[B.i % len(weight_sets)]
            B.i += 1
            check(lib.pg_matmul_quantized_dev(B.h, ptr(acts[k]), M_PREFILL, k, ws[wname], ptr(outs[n]), None))

        settle(one_product)
        prof_one = B.profiled(one_product, 20)[0]
        ours_ms = prof_one["gemm_w8a8"][0]
        # the same clock as the vendor side: stream events around whole calls, less the quantisation launch's kernel time
        ours_stream_ms = B.timed(one_product, 20, 5)["ms_per_step"] - prof_one["quantize_rows"][0]
        entry = {"shape": f"{name}: [{M_PREFILL}x{k}] x [{k}x{n}]", "gemm_w8a8_ms": round(ours_ms, 4),
                 "gemm_w8a8_tops": round(2 * M_PREFILL * k * n / (ours_ms * 1e-3) / 1e12, 1),
                 "gemm_w8a8_stream_event_ms": round(ours_stream_ms, 4)}
        try:
            va = torch.randint(-127, 128, (M_PREFILL, k), dtype=torch.int8, device=dev)
            # as many weight copies in turn as it takes to exceed the 256 MB Infinity Cache: our side streams its
            # weights from HBM too (two weight sets, the f32 activations and the outputs pass through between uses)
            n_rot = max(2, -(-300_000_000 // (k * n)))
            vbs = [torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev).t() for _ in range(n_rot)]

            def vendor_product():
                B.i += 1
                torch._int_mm(va, vbs[B.i % n_rot])

            settle(vendor_product)
            tv = B.timed(vendor_product, 20, 5)
            entry["vendor_int_mm_ms"] = round(tv["ms_per_step"], 4)
            entry["vendor_int_mm_min_ms"] = round(tv["min_ms"], 4)
            entry["vendor_int_mm_tops"] = round(2 * M_PREFILL * k * n / (tv["ms_per_step"] * 1e-3) / 1e12, 1)
            entry["vendor_weight_copies_rotated"] = n_rot
            del va, vbs
        except Exception as exc:  # the calibration is optional
            entry["vendor_int_mm_error"] = repr(exc)[:120]
        vendor.append(entry)

    line = {
        "metric": METRIC, "value": round(tops, 2), "unit": "TOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "median_ms": round(t_head["median_ms"], 4),
        "min_ms": round(t_head["min_ms"], 4), "std_ms": round(t_head["std_ms"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic (the reference's Philox 4x32-10 / Xoshiro256++ Box-Muller generators restated, fixed seeds)",
        "config": {"workload": "cfg3: W8A8 prefill GEMMs of one Llama-3-8B layer at M=2048 "
                               "(q 4096->4096, k/v 4096->1024, o 4096->4096, gate/up 4096->14336, down 14336->4096; q|k|v and gate|up "
                               "as fused products, four calls), "
                               "activations N(0,1) with 1% channels x20, weights N(0,0.02), two weight sets (436 MB) alternated so that they stream from HBM, "
                               "each call = per-row activation quantisation + i8 GEMM + f32 rescale",
                   "m": M_PREFILL, "ops_per_step": LAYER_OPS, "untimed_settle_s": SETTLE_S},
        "pct_int8_mfma_peak": round(100 * tops / PEAK_INT8_TOPS, 2),
        "roofline": roofline, "ceilings": ceil, "gemm_vs_vendor_library": vendor, "activation_quant": act_quant,
    }

    # keep one set of device-quantised weights on the host for the CPU baseline
    cpu_w, cpu_a = {}, {}
    if B.cpu:
        for name, k, n in LAYER:
            qt = np.empty(k * n, np.int8)
            sc = np.empty(n, np.float32)
            check(lib.pg_qtensor_download(B.h, weights[name], None, C.c_void_p(qt.ctypes.data),
                                          C.c_void_p(sc.ctypes.data)))
            cpu_w[name] = (qt, sc)
        cpu_a = {k: acts[k][:CPU_ROWS].cpu().numpy().copy() for k in acts}

    if not args.only_headline:
        # ---- W8A32 (the reference's GPU numerics), gate product
        def w8a32_step():
            check(lib.pg_matmul_dequant_i8_dev(B.h, ptr(acts[4096]), M_PREFILL, 4096, weights["gate_proj"], ptr(outs[14336])))

        t32 = B.timed(w8a32_step, args.steps, args.warmup)
        prof32, _ = B.profiled(w8a32_step, args.steps)
        line["w8a32_gate"] = {"workload": "W8A32 product [2048x4096] x [4096x14336] (f32 activations, dequantised i8 weights, f32 accumulate): "
                                          "three int8 digit planes of 24-bit fixed-point activations: the two low planes as one matrix-core launch, the high plane's launch finishes the sum in its epilogue",
                              "value": round(2 * M_PREFILL * 4096 * 14336 / (t32["ms_per_step"] * 1e-3) / 1e12, 1), "unit": "TFLOP/s",
                              **B.stats(t32, 4), "kernels_ms": {k: round(v[0], 5) for k, v in prof32.items()}}
    for ws in weight_sets:
        for name, _, _ in LAYER:
            lib.pg_qtensor_free(B.h, ws[name])
    del acts, outs
    torch.cuda.empty_cache()

    if not args.only_headline:
        section_decode_and_linear(B, line)
        section_reference_shapes(B, line)
        section_gguf(B, line)
        section_gguf_many_rows(B, line)
        section_mxfp4(B, line)
        section_moe(B, line)
        section_llama_block(B, line)
        section_decode_attention(B, line)
        section_huffman(B, line)
        section_huffman_kv(B, line)

    if args.calibrate_copy:  # a plain copy of known size: 512 MiB read + 512 MiB written per launch
        src = torch.empty(128 << 20, device=dev, dtype=torch.float32).normal_()
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    line["launch_work_items"] = LAUNCHES_SEEN
    line["cpu_baseline"] = cpu_baseline(B.orc, cpu_w, cpu_a) if B.cpu else None
    print(json.dumps(line), flush=True)
    B.ctx.close()


def probe_shapes(B):
    """What a launch that does nothing but read N bytes reaches, by launch shape: GB/s for every (workgroups, threads
    per workgroup, 128-bit loads in flight per lane) at the byte counts of cfg4's product (33 MB), cfg2's down (59 MB)
    and cfg2's gate|up (118 MB); the buffers are rotated so that neither the L2s nor the Infinity Cache serve them."""
    out = {"what": " ".join(probe_shapes.__doc__.split()), "unit": "GB/s", "rows": []}
    for label, nbytes, bufs in (("33MB", 33103872, 10), ("59MB", 58851328, 6), ("118MB", 117702656, 4)):
        for wgs in (256, 512, 1024, 2048, 4096):
            for thr in (256, 512, 1024):
                for inflight in (4, 8, 16):
                    g = C.c_double()
                    B.check(B.lib.pg_probe_hbm_read_shaped(B.h, nbytes, bufs, 200, wgs, thr, inflight, C.byref(g)))
                    out["rows"].append([label, wgs, thr, inflight, round(g.value, 1)])
    return out


def cache_residency(B):
    """How much of a one-row product's time is the weight stream?  The same product over 1, 2, 3, 4, 6 and 12
    tensors used in turn: one 33 MB tensor is served by the eight L2s (4 MB each), 66 - 198 MB by the 256 MB
    Infinity Cache, 396 MB and more by HBM.  us per product (stream time over 240 products, launches included)."""
    import numpy as np

    torch, lib, check, ptr, dev, _ffi = B.torch, B.lib, B.check, B.ptr, B.dev, B.ffi
    rots = (1, 2, 3, 4, 6, 12)
    out = {"what": cache_residency.__doc__.split("  us per")[0].replace("\n   ", ""), "unit": "us per product", "tensors_rotated": list(rots)}

    def sweep(step_for):
        row = []
        for rot in rots:
            B.i = 0
            t = B.timed(step_for(rot), 240, 48)
            row.append(round(t["ms_per_step"] * 1e3, 2))
        return row

    for n_out, k_in in ((14336, 4096), (4096, 14336), (28672, 4096)):
        raw = np.frombuffer(B.synth.pack_q4_0(B.normal(7300 + n_out % 97, (n_out, k_in), 0.02).cpu().numpy()), np.uint8)
        hs = []
        for _ in range(max(rots)):
            h = C.c_void_p()
            check(lib.pg_gguf_upload(B.h, C.c_void_p(raw.ctypes.data), _ffi.GGML_Q4_0, n_out, k_in, C.byref(h)))
            hs.append(h)
        x, y = B.make_acts(1, k_in, 1250), torch.empty(1, n_out, device=dev)

        def step_for(rot):
            def step():
                check(lib.pg_gguf_matmul_dev(B.h, ptr(x), 1, hs[B.i % rot], ptr(y)))
                B.i += 1
            return step
        out[f"q4_0 [{k_in}]->[{n_out}] ({raw.size / 1e6:.0f} MB each)"] = sweep(step_for)
        for h in hs:
            lib.pg_gguf_free(B.h, h)
    for k, n in ((4096, 14336), (14336, 4096)):
        ws = [B.make_weight(k, n, 7400 + i) for i in range(max(rots))]
        x, y = B.make_acts(1, k, 1251), torch.empty(1, n, device=dev)

        def step_for(rot):
            def step():
                check(lib.pg_matmul_quantized_dev(B.h, ptr(x), 1, k, ws[B.i % rot], ptr(y), None))
                B.i += 1
            return step
        out[f"int8 [{k}]->[{n}] ({k * n / 1e6:.0f} MB each)"] = sweep(step_for)
        for h in ws:
            lib.pg_qtensor_free(B.h, h)
    return out


def section_decode_and_linear(B, line):
    """cfg2 (M = 1 int8 GEMV at the FFN shapes) and cfg1 (one W8A8 linear at M = 32)."""
    torch, lib, check, ptr, dev, args = B.torch, B.lib, B.check, B.ptr, B.dev, B.args
    LAYERS_ROT = 4  # 4 x (gate, up, down) = 704 MB of distinct weights > 256 MB Infinity Cache
    kept = []  # the first layer's f32 weights, for the CPU baseline
    dec_w = []
    for r in range(LAYERS_ROT):
        keep = kept if (r == 0 and B.cpu) else None
        dec_w.append((B.make_weight(4096, 14336, 7000 + 3 * r, keep), B.make_weight(4096, 14336, 7001 + 3 * r, keep),
                      B.make_weight(14336, 4096, 7002 + 3 * r, keep)))
    x_d, x_f = B.make_acts(1, 4096, 1240), B.make_acts(1, 14336, 1242)
    y_f, y_u, y_d = torch.empty(1, 14336, device=dev), torch.empty(1, 14336, device=dev), torch.empty(1, 4096, device=dev)

    VP2 = C.c_void_p * 2
    gu_tabs = [VP2(g.value, u.value) for g, u, _ in dec_w]
    gu_out = VP2(y_f.data_ptr(), y_u.data_ptr())

    def decode_step():  # gate|up as the fused product of models::llama (one launch), then down
        r = B.i % LAYERS_ROT
        B.i += 1
        check(lib.pg_matmul_quantized_multi_dev(B.h, ptr(x_d), 1, 4096, gu_tabs[r], 2, gu_out))
        check(lib.pg_matmul_quantized_dev(B.h, ptr(x_f), 1, 14336, dec_w[r][2], ptr(y_d), None))

    dec_bytes = 2 * gemv_bytes(4096, 14336) + gemv_bytes(14336, 4096)
    t_dec = B.timed(decode_step, B.dsteps, max(args.warmup, 8))
    prof, grids = B.profiled(decode_step, B.dsteps)
    gemv_avg_ms, v_n = prof["gemv_w8a8"]
    gemv_lps = v_n / B.dsteps  # launches per step: gate|up together, down
    gemv_gbs = (dec_bytes / gemv_lps) / (gemv_avg_ms * 1e-3) / 1e9
    decode = {"workload": "cfg2: M=1 int8 GEMV, x[4096]->gate|up[14336+14336] (one launch), x[14336]->down[4096]; "
                          f"{LAYERS_ROT} layers of weights rotated ({LAYERS_ROT * 3 * 58.7:.0f} MB, HBM-resident reads)",
              "value": round(dec_bytes / (t_dec["ms_per_step"] * 1e-3) / 1e9, 1), "unit": "GB/s",
              "frac_of_hbm_peak": round(dec_bytes / (t_dec["ms_per_step"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
              **B.stats(t_dec), "steps": B.dsteps, "bytes_per_step": dec_bytes,
              "roofline": {"kernel": "gemv_w8a8_m1_f32x_kernel (quantises its activation row, then streams the weights)", "bound": "hbm",
                           "achieved": round(gemv_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gemv_gbs / PEAK_HBM_GBS, 4),
                           "traffic": B.traffic_for("gemv_w8a8", grids), "bytes_per_launch": int(dec_bytes / gemv_lps),
                           "launches_per_step": gemv_lps, "avg_launch_ms": round(gemv_avg_ms, 5)}}
    if B.cpu:
        decode["cpu_baseline"] = cpu_decode(B.orc, kept, x_d.cpu().numpy(), x_f.cpu().numpy(), dec_bytes)
    # the same step over a small batch of rows (batched decode): the rows are quantised once, then one launch per weight
    batched = []
    for rows in (8, 32):
        xb_d, xb_f = B.make_acts(rows, 4096, 1244), B.make_acts(rows, 14336, 1245)
        yb_f, yb_u, yb_d = (torch.empty(rows, n, device=dev) for n in (14336, 14336, 4096))
        gub_out = VP2(yb_f.data_ptr(), yb_u.data_ptr())

        def batch_step():
            r = B.i % LAYERS_ROT
            B.i += 1
            check(lib.pg_matmul_quantized_multi_dev(B.h, ptr(xb_d), rows, 4096, gu_tabs[r], 2, gub_out))
            check(lib.pg_matmul_quantized_dev(B.h, ptr(xb_f), rows, 14336, dec_w[r][2], ptr(yb_d), None))

        t_b = B.timed(batch_step, B.dsteps, max(args.warmup, 8))
        prof_b, _ = B.profiled(batch_step, B.dsteps)
        batched.append({"rows": rows, "ms_per_step": round(t_b["ms_per_step"], 5), "weight_gbs": round(3 * 4096 * 14336 / (t_b["ms_per_step"] * 1e-3) / 1e9, 1),
                        "kernels_ms_x_launches": {k: [round(v[0], 5), v[1] / B.dsteps] for k, v in prof_b.items()}})
    decode["batched"] = batched
    line["decode_gemv"] = decode
    del kept
    for trio in dec_w:
        for h in trio:
            lib.pg_qtensor_free(B.h, h)
    torch.cuda.empty_cache()

    # ---- cfg1: one W8A8 linear, M = 32
    keep1 = [] if B.cpu else None
    w1 = [B.make_weight(4096, 4096, 7100 + i, keep1 if i == 0 else None) for i in range(8)]  # 8 x 16.8 MB rotated
    a1 = B.normal(1250, (32, 4096))
    o1 = torch.empty(32, 4096, device=dev)

    def lin_step():
        h = w1[B.i % len(w1)]
        B.i += 1
        check(lib.pg_matmul_quantized_dev(B.h, ptr(a1), 32, 4096, h, ptr(o1), None))

    t_lin = B.timed(lin_step, B.dsteps, max(args.warmup, 8))
    prof, _ = B.profiled(lin_step, B.dsteps)
    lin_bytes = 17842176
    linear_m32 = {"workload": "cfg1: W8A8 linear [32x4096] x [4096x4096] (the reference's CPU-runnable case); 8 weights rotated",
                  "value": round(2 * 32 * 4096 * 4096 / (t_lin["ms_per_step"] * 1e-3) / 1e12, 2), "unit": "TOP/s",
                  "gbs": round(lin_bytes / (t_lin["ms_per_step"] * 1e-3) / 1e9, 1), **B.stats(t_lin),
                  "kernels_ms": {k: round(v[0], 5) for k, v in prof.items()}}
    if B.cpu:
        linear_m32["cpu_baseline"] = cpu_linear(B.orc, keep1[0], a1.cpu().numpy())
    line["linear_m32"] = linear_m32
    for h in w1:
        lib.pg_qtensor_free(B.h, h)
    torch.cuda.empty_cache()


def section_reference_shapes(B, line):
    """The two int8 products the reference's own benchmark times (benches/wallclock.rs:758-786: `matmul_i8_196x768x3072`,
    `matmul_i8_196x1024x4096`, ViT FFN shapes; 5 warm-up + 20 timed calls, median, :19-41), through the device entry point
    (operands resident) and through the host-pointer entry point (what `Tensor::matmul_quantized` on host slices costs:
    PCIe both ways inside the call), with the CPU oracle beside them."""
    import numpy as np

    torch, lib, check, ptr, dev = B.torch, B.lib, B.check, B.ptr, B.dev
    published = {"196x768x3072": 12060.2, "196x1024x4096": 21728.7}  # us, M1 Max CPU medians (benchmarks/BENCHMARKS.md:234,236)
    rows = []
    for m, k, n in ((196, 768, 3072), (196, 1024, 4096)):
        label = f"{m}x{k}x{n}"
        a = B.normal(7300 + k, (m, k))          # Tensor::randn: N(0, 1) for both operands
        w = B.normal(7301 + k, (k, n))
        h = C.c_void_p()
        check(lib.pg_qtensor_from_f32_dev(B.h, ptr(w), k, n, C.byref(h)))
        out = torch.empty(m, n, device=dev)

        def dev_call():
            check(lib.pg_matmul_quantized_dev(B.h, ptr(a), m, k, h, ptr(out), None))

        t_dev = B.timed(dev_call, 20, 5)
        prof, _ = B.profiled(dev_call, 20)
        a_h = a.cpu().numpy().copy()
        out_h = np.empty((m, n), np.float32)

        def host_call():
            check(lib.pg_matmul_quantized(B.h, C.c_void_p(a_h.ctypes.data), m, k, h, C.c_void_p(out_h.ctypes.data)))

        for _ in range(5):
            host_call()
        wall = []
        for _ in range(20):
            t0 = time.perf_counter()
            host_call()
            wall.append((time.perf_counter() - t0) * 1e6)
        row = {"name": f"matmul_i8_{label}", "ops": 2 * m * k * n,
               "device_entry_median_us": round(t_dev["median_ms"] * 1e3, 2), "device_entry_min_us": round(t_dev["min_ms"] * 1e3, 2),
               "device_entry_tops": round(2 * m * k * n / (t_dev["median_ms"] * 1e-3) / 1e12, 2),
               "kernels_us": {kk: round(v[0] * 1e3, 2) for kk, v in prof.items()},
               "host_entry_median_us": round(statistics.median(wall), 1), "host_entry_min_us": round(min(wall), 1),
               "reference_published_median_us": published[label]}
        if B.cpu:
            olib = B.orc["lib"]
            qt_i8, sc = _cpu_quantize(olib, w.cpu().numpy())
            ref_out = np.empty((m, n), np.float32)

            def cpu_call():
                olib.orc_matmul_quantized(_vp(a_h), C.c_size_t(m), C.c_size_t(k), _vp(qt_i8), _vp(sc), C.c_size_t(n), _vp(ref_out), None)

            cpu_call()
            row["cpu_oracle_us"] = round(_best_of(cpu_call, 3) * 1e6, 1)
            row["bit_equal_to_cpu_oracle"] = bool((ref_out.view(np.uint32) == out_h.view(np.uint32)).all())
        rows.append(row)
        lib.pg_qtensor_free(B.h, h)
    line["reference_bench_shapes"] = {
        "what": "the reference's own int8 benchmark (benches/wallclock.rs:758-786), its protocol (5 warm-up + 20 timed, median); "
                "`reference_published_median_us` is the reference's published CPU figure on an M1 Max, quoted as context, not a like-for-like baseline",
        "rows": rows, "cpu_oracle": "scalar C restatement of src/quant.rs:129-169, one thread of this host" if B.cpu else None}


def section_gguf(B, line):
    """cfg4: the Q4_0 dequant-matmul [4096] -> [14336] at M = 1 (streaming GEMV), 4 and 16 (matrix cores)."""
    import numpy as np

    torch, lib, check, ptr, dev, args, _ffi = B.torch, B.lib, B.check, B.ptr, B.dev, B.args, B.ffi
    n_out, k_in = 14336, 4096
    wq = B.normal(7200, (n_out, k_in), 0.02).cpu().numpy()
    raw = np.frombuffer(B.synth.pack_q4_0(wq), np.uint8)
    del wq
    Q4_ROT = 10  # 10 x 33 MB = 330 MB of distinct Q4_0 tensors
    q4 = []
    for _ in range(Q4_ROT):
        h = C.c_void_p()
        check(lib.pg_gguf_upload(B.h, C.c_void_p(raw.ctypes.data), _ffi.GGML_Q4_0, n_out, k_in, C.byref(h)))
        q4.append(h)
    x_1 = B.make_acts(1, k_in, 1240)
    y_q = torch.empty(1, n_out, device=dev)

    def q4_step():
        h = q4[B.i % Q4_ROT]
        B.i += 1
        check(lib.pg_gguf_matmul_dev(B.h, ptr(x_1), 1, h, ptr(y_q)))

    q4_bytes = n_out * (k_in // 32) * 18 + 4 * k_in + 4 * n_out  # 33 103 872
    t_q4 = B.timed(q4_step, B.dsteps, max(args.warmup, 8))
    prof, grids = B.profiled(q4_step, B.dsteps)
    q4_avg_ms, k_n = prof["gguf_gemv_q4_0"]
    q4_gbs = q4_bytes / (q4_avg_ms * 1e-3) / 1e9
    gguf = {"workload": f"cfg4: M=1 Q4_0 dequant-GEMV [4096]->[14336]; {Q4_ROT} tensors rotated (330 MB)",
            "value": round(q4_bytes / (t_q4["ms_per_step"] * 1e-3) / 1e9, 1), "unit": "GB/s",
            "frac_of_hbm_peak": round(q4_bytes / (t_q4["ms_per_step"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), **B.stats(t_q4),
            "kernels_ms": {k: round(v[0], 5) for k, v in prof.items()},
            "roofline": {"kernel": "gguf_gemv_kernel<Q4_0>", "bound": "hbm", "achieved": round(q4_gbs, 1),
                         "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(q4_gbs / PEAK_HBM_GBS, 4),
                         "traffic": B.traffic_for("gguf_gemv_q4_0", grids), "bytes_per_launch": q4_bytes,
                         "avg_launch_ms": round(q4_avg_ms, 5)}}
    cpu_q4 = cpu_gguf(B.orc, raw, n_out, k_in, (1, 4, 16)) if B.cpu else {}
    if B.cpu:
        gguf["cpu_baseline"] = cpu_q4[1]
    line["gguf_q4_0_gemv"] = gguf
    skinny = []
    for m_q in (4, 16):
        x_m = B.normal(1260 + m_q, (m_q, k_in))
        y_m = torch.empty(m_q, n_out, device=dev)

        def mm_step():
            h = q4[B.i % Q4_ROT]
            B.i += 1
            check(lib.pg_gguf_matmul_dev(B.h, ptr(x_m), m_q, h, ptr(y_m)))

        mm_bytes = n_out * (k_in // 32) * 18 + 4 * m_q * k_in + 4 * m_q * n_out
        t_mm = B.timed(mm_step, B.dsteps, max(args.warmup, 8))
        prof, grids = B.profiled(mm_step, B.dsteps)
        # up to 8 rows: one matrix-core launch after the digits (gguf_skinny_kernel); more: product over K chunks + their sum
        k_name = "gguf_q4_0_few_rows_mm" if "gguf_q4_0_few_rows_mm" in prof else "gguf_mm_q4_0"
        k_ms = prof[k_name][0]
        entry = {"workload": f"cfg4: M={m_q} Q4_0 dequant-matmul [{m_q}x4096]->[{m_q}x14336], weights read once",
                 "value": round(mm_bytes / (t_mm["ms_per_step"] * 1e-3) / 1e9, 1), "unit": "GB/s", **B.stats(t_mm),
                 "gflops": round(2 * m_q * n_out * k_in / (t_mm["ms_per_step"] * 1e-3) / 1e9, 1),
                 "kernels_ms": {k: round(v[0], 5) for k, v in prof.items()},
                 "roofline": {"kernel": "gguf_skinny_kernel<Q4_0>" if k_name == "gguf_q4_0_few_rows_mm" else "gguf_mm_kernel<Q4_0>", "bound": "hbm",
                              "achieved": round(mm_bytes / (k_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                              "frac": round(mm_bytes / (k_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                              "traffic": B.traffic_for(k_name, grids),
                              "bytes_per_launch": mm_bytes, "avg_launch_ms": round(k_ms, 5)}}
        if B.cpu:
            entry["cpu_baseline"] = cpu_q4[m_q]
        skinny.append(entry)
    line["gguf_q4_0_skinny"] = skinny
    # the same tensors at the other small row counts (a few draft tokens being verified): whole call, digits' launch included
    other = []
    for m_q in (2, 3, 8, 12):
        x_m = B.normal(1270 + m_q, (m_q, k_in))
        y_m = torch.empty(m_q, n_out, device=dev)

        def mm_step():
            h = q4[B.i % Q4_ROT]
            B.i += 1
            check(lib.pg_gguf_matmul_dev(B.h, ptr(x_m), m_q, h, ptr(y_m)))

        t_mm = B.timed(mm_step, B.dsteps, max(args.warmup, 8))
        other.append({"rows": m_q, "ms_per_step": round(t_mm["ms_per_step"], 5),
                      "weight_gbs": round(n_out * (k_in // 32) * 18 / (t_mm["ms_per_step"] * 1e-3) / 1e9, 1)})
    line["gguf_q4_0_other_row_counts"] = other
    for h in q4:
        lib.pg_gguf_free(B.h, h)
    torch.cuda.empty_cache()


def section_gguf_many_rows(B, line):
    """Row (a) at prefill size: 1024 rows through the Q4_0 dequant-matmul [4096] -> [14336] (a Llama-3-8B gate
    projection).  The dispatcher's route (f16 matrix cores, weights exact) and, forced, the int8 block product."""
    import numpy as np

    torch, lib, check, ptr, dev, _ffi = B.torch, B.lib, B.check, B.ptr, B.dev, B.ffi
    n_out, k_in, m = 14336, 4096, 1024
    raw = np.frombuffer(B.synth.pack_q4_0(B.normal(7210, (n_out, k_in), 0.02).cpu().numpy()), np.uint8)
    hs = []
    for _ in range(8):  # 8 x 33 MB: past the Infinity Cache
        h = C.c_void_p()
        check(lib.pg_gguf_upload(B.h, C.c_void_p(raw.ctypes.data), _ffi.GGML_Q4_0, n_out, k_in, C.byref(h)))
        hs.append(h)
    x = B.make_acts(m, k_in, 1290)
    y = torch.empty(m, n_out, device=dev)

    def step():
        check(lib.pg_gguf_matmul_dev(B.h, ptr(x), m, hs[B.i % len(hs)], ptr(y)))
        B.i += 1

    flop = 2 * m * n_out * k_in
    t = B.timed(step, 24, 8)
    prof, grids = B.profiled(step, 16)
    k_ms = prof["gguf_hmm_q4_0"][0]
    check(lib.pg_gguf_hmm_force(B.h, 2))
    try:
        t_i8 = B.timed(step, 24, 8)
        prof_i8, _ = B.profiled(step, 16)
    finally:
        check(lib.pg_gguf_hmm_force(B.h, 0))
    entry = {"workload": f"row (a), prefill size: Q4_0 dequant-matmul [{m}x{k_in}]->[{m}x{n_out}]; {len(hs)} tensors rotated",
             "value": round(flop / (t["ms_per_step"] * 1e-3) / 1e12, 1), "unit": "TFLOP/s", **B.stats(t),
             "kernels_ms": {k: round(v[0], 5) for k, v in prof.items()},
             "roofline": {"kernel": "gguf_hmm_kernel<Q4_0, 2, 4> (v_mfma_f32_16x16x32_f16; weights unpacked exactly in registers, "
                                    "activations as two f16 planes: twice the counted flops run on the matrix cores)",
                          "bound": "mfma", "achieved": round(flop / (k_ms * 1e-3) / 1e12, 1), "peak": 2500.0, "unit": "TFLOP/s",
                          "frac": round(flop / (k_ms * 1e-3) / 1e12 / 2500.0, 4), "executed_tflops": round(2 * flop / (k_ms * 1e-3) / 1e12, 1),
                          "traffic": B.traffic_for("gguf_hmm_q4_0", grids), "flop_per_launch": flop, "avg_launch_ms": round(k_ms, 5)},
             "int8_block_route": {"ms_per_step": t_i8["ms_per_step"], "tflops": round(flop / (t_i8["ms_per_step"] * 1e-3) / 1e12, 1),
                                  "kernels_ms": {k: round(v[0], 5) for k, v in prof_i8.items()}}}
    if B.cpu:
        rows = 4
        xs = x[:rows].cpu().numpy()
        want = np.empty(rows * n_out, np.float32)
        olib = B.orc["lib"]

        def run():
            assert olib.orc_gguf_matmul(_vp(xs), C.c_size_t(rows), _vp(raw), C.c_int(_ffi.GGML_Q4_0), C.c_size_t(n_out), C.c_size_t(k_in), _vp(want)) == 0

        dt = _best_of(run, 1)
        step()  # (the dispatcher's route again: y held the forced run's result)
        torch.cuda.synchronize()
        got = y[:rows].cpu().numpy().reshape(rows, n_out).astype(np.float64)
        ref = want.reshape(rows, n_out).astype(np.float64)
        floor = np.sqrt((ref * ref).mean(axis=1, keepdims=True))
        entry["max_error_vs_cpu_oracle"] = float(f"{(np.abs(got - ref) / np.maximum(np.abs(ref), floor)).max():.3e}")
        entry["cpu_baseline"] = {"value": round(2 * rows * n_out * k_in / dt / 1e12, 5), "unit": "TFLOP/s", "ms": round(dt * 1e3, 1), "cores": 1,
                                 "kind": "port", "sample": f"{rows} of the {m} rows through the oracle's dequantise -> f32 product "
                                                           f"(linear in the rows), single thread, gcc {B.orc['flags']}"}
    line["gguf_q4_0_many_rows"] = entry
    for h in hs:
        lib.pg_gguf_free(B.h, h)
    torch.cuda.empty_cache()


def section_mxfp4(B, line):
    """MXFP4 one-row products (examples/gpt_oss/moe.rs mxfp4_matmul): the gpt-oss expert shapes and cfg4's shape."""
    import numpy as np

    torch, lib, check, ptr, dev, args = B.torch, B.lib, B.check, B.ptr, B.dev, B.args
    out = []
    rng = np.random.default_rng(7400)
    for n_out, k_in, rot in ((14336, 4096, 10), (5760, 2880, 40), (2880, 2880, 80)):
        codes = rng.integers(0, 256, size=n_out * k_in // 2, dtype=np.uint8)
        scales = rng.integers(118, 124, size=n_out * k_in // 32, dtype=np.uint8)
        hs = []
        for r in range(rot):  # rot x 17 B per block of distinct tensors: more than the 256 MB last-level cache
            codes[0] = r
            h = C.c_void_p()
            check(lib.pg_mxfp4_upload(B.h, C.c_void_p(codes.ctypes.data), C.c_void_p(scales.ctypes.data), n_out, k_in, C.byref(h)))
            hs.append(h)
        x = B.make_acts(1, k_in, 7410)
        y = torch.empty(1, n_out, device=dev)

        def step():
            h = hs[B.i % rot]
            B.i += 1
            check(lib.pg_gguf_matmul_dev(B.h, ptr(x), 1, h, ptr(y)))

        nbytes = n_out * (k_in // 32) * 17 + 4 * k_in + 4 * n_out
        t = B.timed(step, B.dsteps, max(args.warmup, 8))
        prof, grids = B.profiled(step, B.dsteps)
        k_ms = prof["mxfp4_rows"][0]
        out.append({"workload": f"M=1 MXFP4 [{k_in}]->[{n_out}], one launch (FP4 codes and E8M0 scales straight into the scaled "
                                f"matrix-core instruction); {rot} tensors rotated",
                    "value": round(nbytes / (t["ms_per_step"] * 1e-3) / 1e9, 1), "unit": "GB/s",
                    "frac_of_hbm_peak": round(nbytes / (t["ms_per_step"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), **B.stats(t),
                    "roofline": {"kernel": "mxfp4_rows_kernel", "bound": "hbm", "achieved": round(nbytes / (k_ms * 1e-3) / 1e9, 1),
                                 "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(nbytes / (k_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                                 "traffic": B.traffic_for("mxfp4_rows", grids), "bytes_per_launch": nbytes,
                                 "avg_launch_ms": round(k_ms, 5)}})
        for h in hs:
            lib.pg_gguf_free(B.h, h)
    line["mxfp4_gemv"] = out
    torch.cuda.empty_cache()

    # many rows: the tile kernel on the same instruction (prefill-sized, and the gpt-oss expert shapes at 128 tokens)
    many = []
    for m, n_out, k_in in ((1024, 14336, 4096), (1024, 4096, 14336), (128, 5760, 2880), (128, 2880, 2880)):
        codes = rng.integers(0, 256, size=n_out * k_in // 2, dtype=np.uint8)
        scales = rng.integers(118, 124, size=n_out * k_in // 32, dtype=np.uint8)
        hs = []
        for r in range(4):
            codes[0] = r
            h = C.c_void_p()
            check(lib.pg_mxfp4_upload(B.h, C.c_void_p(codes.ctypes.data), C.c_void_p(scales.ctypes.data), n_out, k_in, C.byref(h)))
            hs.append(h)
        x = B.make_acts(m, k_in, 7420)
        y = torch.empty(m, n_out, device=dev)

        def step():
            h = hs[B.i % 4]
            B.i += 1
            check(lib.pg_gguf_matmul_dev(B.h, ptr(x), m, h, ptr(y)))

        t = B.timed(step, B.dsteps, max(args.warmup, 8))
        prof, grids = B.profiled(step, B.dsteps)
        flop = 2.0 * m * n_out * k_in
        k_ms = prof["mxfp4_tiles"][0]
        many.append({"workload": f"MXFP4 [{m} x {k_in}] -> [{n_out}]: activation rows as four planes of E4M3 base-32 digits, "
                                 f"FP4 codes and both sides' block scales inside v_mfma_scale_f32_16x16x128_f8f6f4",
                     "value": round(flop / (t["ms_per_step"] * 1e-3) / 1e12, 1), "unit": "TFLOP/s", **B.stats(t),
                     "kernels_ms": {k: round(v[0], 5) for k, v in prof.items()},
                     "roofline": {"kernel": "mxfp4_tiles_kernel", "bound": "mfma", "achieved": round(flop / (k_ms * 1e-3) / 1e12, 1),
                                  "peak": 5000.0, "unit": "TFLOP/s", "frac": round(flop / (k_ms * 1e-3) / 1e12 / 5000.0, 4),
                                  "executed_tflops": round(4 * flop / (k_ms * 1e-3) / 1e12, 1), "traffic": B.traffic_for("mxfp4_tiles", grids) if not many else None,
                                  "avg_launch_ms": round(k_ms, 5),
                                  "note": "peak = the published dense FP8 rate (an FP4 x FP8 instruction runs at it); "
                                          "executed = four digit planes per algorithmic multiply-add"}})
        for h in hs:
            lib.pg_gguf_free(B.h, h)
    line["mxfp4_many_rows"] = many
    torch.cuda.empty_cache()

    # the gpt-oss-20b MoE layer after its router: 32 MXFP4 experts (hidden = intermediate = 2880), top 4
    hidden = inter = 2880
    E, top_k = 32, 4
    experts = []
    for e in range(E):
        b1 = rng.integers(0, 256, size=2 * inter * hidden // 2, dtype=np.uint8)
        s1 = rng.integers(118, 124, size=2 * inter * hidden // 32, dtype=np.uint8)
        b2 = rng.integers(0, 256, size=hidden * inter // 2, dtype=np.uint8)
        s2 = rng.integers(118, 124, size=hidden * inter // 32, dtype=np.uint8)
        bias1 = rng.standard_normal(2 * inter).astype(np.float32)
        bias2 = rng.standard_normal(hidden).astype(np.float32)
        h = C.c_void_p()
        check(lib.pg_mxfp4_expert_create(B.h, hidden, inter, C.c_float(1.702), C.c_float(7.0), C.c_void_p(b1.ctypes.data), C.c_void_p(s1.ctypes.data),
                                         C.c_void_p(b2.ctypes.data), C.c_void_p(s2.ctypes.data), C.c_void_p(bias1.ctypes.data),
                                         C.c_void_p(bias2.ctypes.data), C.byref(h)))
        experts.append(h)
    tab = (C.c_void_p * E)(*[h.value for h in experts])
    weight_bytes = E * 3 * inter * (hidden // 32) * 17
    moe = []
    for T in (1024, 1):
        x = B.make_acts(T, hidden, 7430)
        logits = B.normal(7431, (T, E), 1.0)
        top = torch.topk(logits, top_k, dim=1)
        idx = top.indices.to(torch.int32).contiguous()
        wt = torch.softmax(top.values, dim=1).contiguous()
        out = torch.empty(T, hidden, device=dev)
        torch.cuda.synchronize()

        def step():
            check(lib.pg_mxfp4_moe_ffn_routed_dev(B.h, ptr(x), T, ptr(idx), ptr(wt), top_k, C.cast(tab, C.POINTER(C.c_void_p)), E, ptr(out)))

        t = B.timed(step, B.dsteps, max(args.warmup, 8))
        prof, _ = B.profiled(step, B.dsteps)
        # the same layer as the reference walks it, batched per expert: one Mxfp4Expert::forward per expert over its tokens
        lists = [torch.nonzero((idx == e).any(dim=1)).flatten() for e in range(E)]
        xs = [x[l].contiguous() for l in lists]
        scratch = torch.empty(max(1, max(l.numel() for l in lists)) * 3 * inter, device=dev)
        outs = [torch.empty(max(1, l.numel()), hidden, device=dev) for l in lists]

        def loop_step():
            for e in range(E):
                if lists[e].numel():
                    check(lib.pg_mxfp4_expert_forward_dev(B.h, experts[e], ptr(xs[e]), lists[e].numel(), ptr(scratch), ptr(outs[e])))

        tl = B.timed(loop_step, max(3, B.dsteps // 4), 3)
        flop = 2.0 * T * top_k * 3 * inter * hidden
        touched = min(E, T * top_k) / E * weight_bytes if T == 1 else weight_bytes
        entry = {"workload": f"gpt-oss-20b MoE layer after its router: {T} token(s), {E} MXFP4 experts of {hidden} -> 2 x {inter} -> {hidden}, top {top_k}; "
                             f"routing from N(0,1) logits (top-k, softmax over the k)",
                 "ms_per_step": round(t["ms_per_step"], 5), **B.stats(t),
                 "value": round(flop / (t["ms_per_step"] * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
                 "weights_gbs": round(touched / (t["ms_per_step"] * 1e-3) / 1e9, 1),
                 "per_expert_calls_ms": round(tl["ms_per_step"], 5),
                 "kernels_ms_x_launches": {k: [round(v[0], 5), round(v[1] / B.dsteps, 1)] for k, v in prof.items()}}
        moe.append(entry)
    for h in experts:
        lib.pg_mxfp4_expert_free(B.h, h)
    line["mxfp4_moe_layer"] = moe
    torch.cuda.empty_cache()


def section_moe(B, line):
    """cfg5: Grok-1-shaped MoE expert FFN, Q8_0 experts."""
    torch, lib, check, ptr, dev, _ffi = B.torch, B.lib, B.check, B.ptr, B.dev, B.ffi
    T_moe, d_moe, ffn_moe, E_moe, topk_moe = 64, 6144, 32768, 8, 2
    nblk = ffn_moe * d_moe // 32

    def q8_0_blocks(seed):
        """[ffn x d] ~ N(0, 0.02) quantised to Q8_0 (d = f16(absmax / 127)) on the device; host bytes."""
        w = B.normal(seed, (nblk, 32), 0.02)
        dsc = (w.abs().amax(dim=1) / 127.0).to(torch.float16)
        df = dsc.to(torch.float32)
        safe = torch.where(df > 0, df, torch.ones_like(df))
        q = torch.where(df[:, None] > 0, torch.round(w / safe[:, None]), torch.zeros_like(w)).clamp_(-127, 127).to(torch.int8)
        out = torch.empty(nblk, 34, dtype=torch.uint8, device=dev)
        out[:, :2] = dsc.view(torch.uint8).reshape(nblk, 2)
        out[:, 2:] = q.view(torch.uint8)
        return out.cpu().numpy()

    experts = [[], [], []]
    for which, (no, ki) in enumerate(((ffn_moe, d_moe), (ffn_moe, d_moe), (d_moe, ffn_moe))):
        blocks = q8_0_blocks(7300 + which)  # one quantised matrix per projection, varied per expert below
        torch.cuda.empty_cache()
        for e in range(E_moe):
            blocks[:, 2] = e + 8 * which  # make the tensors differ
            h = C.c_void_p()
            check(lib.pg_gguf_upload(B.h, C.c_void_p(blocks.ctypes.data), _ffi.GGML_Q8_0, no, ki, C.byref(h)))
            experts[which].append(h)
        del blocks
    tabs = [(C.c_void_p * E_moe)(*[h.value for h in experts[w]]) for w in range(3)]
    x_moe = B.normal(1270, (T_moe, d_moe))
    lg_moe = B.normal(1271, (T_moe, E_moe))
    out_moe = torch.empty(T_moe, d_moe, device=dev)

    def moe_step():
        check(lib.pg_moe_ffn_dev(B.h, ptr(x_moe), T_moe, ptr(lg_moe), E_moe, topk_moe, tabs[0], tabs[1], tabs[2],
                                 _ffi.ACT_SILU, ptr(out_moe)))

    moe_bytes = 3 * E_moe * nblk * 34 + 2 * 4 * T_moe * d_moe  # every expert is hit at T=64, k=2 (reported below)
    hit = int(torch.unique(torch.topk(lg_moe, topk_moe, dim=1).indices).numel())
    t_moe = B.timed(moe_step, 20, 10)  # 5 GB of weights: the first passes also warm the TLBs
    prof, grids = B.profiled(moe_step, 5)
    mm_total = prof["gguf_mm_q8_0"][0] * prof["gguf_mm_q8_0"][1] / 5  # three launches per step
    line["moe_q8_0"] = {
        "workload": "cfg5: Grok-1-shaped MoE FFN, Q8_0 experts (d 6144, ffn 32768, 8 experts, top-2, 64 tokens, SiLU); "
                    "5.13 GB of expert weights, read once per step",
        "experts_hit": hit, "value": round(moe_bytes / (t_moe["ms_per_step"] * 1e-3) / 1e9, 1), "unit": "GB/s",
        "frac_of_hbm_peak": round(moe_bytes / (t_moe["ms_per_step"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), **B.stats(t_moe, 4),
        "tflops": round(2 * T_moe * topk_moe * 3 * ffn_moe * d_moe / (t_moe["ms_per_step"] * 1e-3) / 1e12, 2),
        "kernels_ms": {k: round(v[0], 5) for k, v in prof.items()},
        "roofline": {"kernel": "gguf_mm_kernel<Q8_0> (gate, up, down)", "bound": "hbm",
                     "achieved": round(3 * E_moe * nblk * 34 / (mm_total * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(3 * E_moe * nblk * 34 / (mm_total * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                     "traffic": B.traffic_for("gguf_mm_q8_0", grids), "bytes_per_launch": E_moe * nblk * 34,
                     "avg_launch_ms": round(prof["gguf_mm_q8_0"][0], 5)}}
    for w3 in experts:
        for h in w3:
            lib.pg_gguf_free(B.h, h)
    torch.cuda.empty_cache()


def section_decode_attention(B, line):
    """GQA attention of one query token (32 query heads over 8 kv heads of 128, causal) over f32 caches of 1 025 to
    32 769 positions: the bytes are the keys and values, read once."""
    torch, lib, check, ptr, dev = B.torch, B.lib, B.check, B.ptr, B.dev
    nqh, nkv, hd = 32, 8, 128
    out_rows = []
    for ctx_len in (1025, 8193, 32769):
        caches = []
        for r in range(3):  # three caches rotated (0.8 GB at the longest: more than the Infinity Cache)
            kv = C.c_void_p()
            check(lib.pg_kv_cache_create(B.h, nkv, hd, C.byref(kv)))
            k = B.normal(1400 + r, (nkv, ctx_len, hd))
            check(lib.pg_kv_cache_append_dev(B.h, kv, ptr(k), ptr(k), ctx_len))
            caches.append(kv)
            del k
        q = B.normal(1410, (nqh, 1, hd))
        out = torch.zeros(1, nqh * hd, device=dev)

        def step():
            kv = caches[B.i % 3]
            B.i += 1
            check(lib.pg_gqa_attention_dev(B.h, ptr(q), kv, kv, nqh, 1, C.c_float(hd ** -0.5), 1, ctx_len - 1, 0, 0,
                                           C.c_float(0.0), ptr(out)))

        t = B.timed(step, B.dsteps, max(B.args.warmup, 8))
        prof, _ = B.profiled(step, B.dsteps)
        nbytes = 2 * nkv * ctx_len * hd * 4
        k_ms = prof["gqa_decode"][0]
        out_rows.append({"positions": ctx_len, **B.stats(t), "bytes_per_step": nbytes,
                         "value": round(nbytes / (t["ms_per_step"] * 1e-3) / 1e9, 1), "unit": "GB/s",
                         "kernels_ms": {k: round(v[0], 5) for k, v in prof.items()},
                         "roofline": {"kernel": "gqa_decode_kernel<128, U>", "bound": "hbm", "achieved": round(nbytes / (k_ms * 1e-3) / 1e9, 1),
                                      "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(nbytes / (k_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                                      "traffic": None, "bytes_per_launch": nbytes, "avg_launch_ms": round(k_ms, 5)}})
        for kv in caches:
            lib.pg_kv_cache_free(B.h, kv)
        torch.cuda.empty_cache()
    line["decode_attention"] = {"workload": "one query token, 32 / 8 heads of 128, causal, f32 caches; 3 caches rotated", "by_length": out_rows}


def section_llama_block(B, line):
    """One Llama-3-8B decoder block with Q4_0 projections: a one-token step and a 1024-token prefill."""
    import numpy as np

    torch, lib, check, ptr, dev, args, _ffi = B.torch, B.lib, B.check, B.ptr, B.dev, B.args, B.ffi
    d_l, nqh_l, nkv_l, hd_l, ffn_l, ctx_len = 4096, 32, 8, 128, 14336, 1024
    shapes_l = [(nqh_l * hd_l, d_l), (nkv_l * hd_l, d_l), (nkv_l * hd_l, d_l), (d_l, nqh_l * hd_l),
                (ffn_l, d_l), (ffn_l, d_l), (d_l, ffn_l)]
    L_ROT = 4  # 4 x 123 MB of block weights rotated: more than the 256 MB last-level cache
    rng = np.random.default_rng(8)  # block payloads are uniform random nibbles: only the byte count matters here
    blocks_l, keep_l = [], []
    for r in range(L_ROT):
        hs = []
        for no, ki in shapes_l:
            nb = no * ki // 32
            rawb = np.empty((nb, 18), np.uint8)
            rawb[:, 2:] = rng.integers(0, 256, size=(nb, 16), dtype=np.uint8)
            rawb[:, :2] = np.frombuffer(np.float16(0.02 / 7 * 64 / np.sqrt(ki)).tobytes(), np.uint8)
            h = C.c_void_p()
            check(lib.pg_gguf_upload(B.h, C.c_void_p(rawb.ctypes.data), _ffi.GGML_Q4_0, no, ki, C.byref(h)))
            hs.append(h)
        b = C.c_void_p()
        check(lib.pg_llama_block_create(B.h, d_l, nqh_l, nkv_l, hd_l, ffn_l, 4096, 500000.0, 1e-5, C.byref(b)))
        ones = np.ones(d_l, np.float32)
        check(lib.pg_llama_block_set_weights(B.h, b, *hs, C.c_void_p(ones.ctypes.data), C.c_void_p(ones.ctypes.data)))
        kv = C.c_void_p()
        check(lib.pg_kv_cache_create(B.h, nkv_l, hd_l, C.byref(kv)))
        blocks_l.append((b, kv))
        keep_l.append(hs)
    w_bytes_l = sum(no * ki // 32 * 18 for no, ki in shapes_l)
    h_pre = B.normal(1280, (ctx_len, d_l))
    o_pre = torch.empty_like(h_pre)
    h_dec = B.normal(1281, (1, d_l))
    o_dec = torch.empty_like(h_dec)

    def block_prefill():
        b, kv = blocks_l[B.i % L_ROT]
        B.i += 1
        check(lib.pg_kv_cache_rollback_to(kv, 0))
        check(lib.pg_llama_block_forward_dev(B.h, b, ptr(h_pre), ctx_len, kv, ptr(o_pre)))

    def block_decode():  # position ctx_len on top of the prefilled cache, then rolled back
        b, kv = blocks_l[B.i % L_ROT]
        B.i += 1
        check(lib.pg_kv_cache_rollback_to(kv, ctx_len))
        check(lib.pg_llama_block_forward_dev(B.h, b, ptr(h_dec), 1, kv, ptr(o_dec)))

    h_few = B.normal(1282, (4, d_l))
    o_few = torch.empty_like(h_few)

    def block_few():  # four tokens at once on top of the prefilled cache (draft tokens being verified), then rolled back
        b, kv = blocks_l[B.i % L_ROT]
        B.i += 1
        check(lib.pg_kv_cache_rollback_to(kv, ctx_len))
        check(lib.pg_llama_block_forward_dev(B.h, b, ptr(h_few), 4, kv, ptr(o_few)))

    t_pre = B.timed(block_prefill, 16, 8)  # leaves every cache filled to ctx_len
    pre_prof, _ = B.profiled(block_prefill, 8)
    t_bd = B.timed(block_decode, B.dsteps, max(args.warmup, 8))
    dec_prof, _ = B.profiled(block_decode, B.dsteps)
    # (left out of the counter runs: its gate|up launch has the work-items of cfg4's skinny products, and the
    # per-launch-size traffic figures could not tell them apart)
    t_few = B.timed(block_few, B.dsteps, max(args.warmup, 8)) if not args.calibrate_copy else None
    few_prof = B.profiled(block_few, B.dsteps)[0] if not args.calibrate_copy else {}
    kv_bytes_l = 2 * nkv_l * (ctx_len + 1) * hd_l * 4
    dec_bytes_l = w_bytes_l + kv_bytes_l
    pre_flops = 2 * ctx_len * sum(no * ki for no, ki in shapes_l) + 4 * nqh_l * hd_l * ctx_len * (ctx_len + 1) // 2
    line["llama_block_q4_0"] = {
        "workload": f"one Llama-3-8B decoder block (d 4096, 32/8 heads x 128, ffn 14336), Q4_0 projections ({w_bytes_l / 1e6:.0f} MB), "
                    f"f32 KV cache; {L_ROT} blocks rotated",
        "decode": {"what": f"seq 1 at position {ctx_len}", **B.stats(t_bd),
                   "value": round(dec_bytes_l / (t_bd["ms_per_step"] * 1e-3) / 1e9, 1), "unit": "GB/s",
                   "frac_of_hbm_peak": round(dec_bytes_l / (t_bd["ms_per_step"] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                   "bytes_per_step": dec_bytes_l, "launches_per_step": round(sum(v[1] for v in dec_prof.values()) / B.dsteps, 2),
                   "kernels_ms_x_launches": {k: [round(v[0], 5), round(v[1] / B.dsteps, 2)] for k, v in dec_prof.items()}},
        "four_tokens": None if t_few is None else
                       {"what": f"seq 4 at positions {ctx_len}..{ctx_len + 3}", **B.stats(t_few),
                        "launches_per_step": round(sum(v[1] for v in few_prof.values()) / B.dsteps, 2),
                        "kernels_ms_x_launches": {k: [round(v[0], 5), round(v[1] / B.dsteps, 2)] for k, v in few_prof.items()}},
        "prefill": {"what": f"seq {ctx_len} into an empty cache", **B.stats(t_pre, 4),
                    "tflops": round(pre_flops / (t_pre["ms_per_step"] * 1e-3) / 1e12, 1),
                    "tokens_per_s": round(ctx_len / (t_pre["ms_per_step"] * 1e-3), 0),
                    "kernels_ms_x_launches": {k: [round(v[0], 5), round(v[1] / 8, 2)] for k, v in pre_prof.items()}},
    }
    for (b, kv), hs in zip(blocks_l, keep_l):
        lib.pg_llama_block_free(B.h, b)
        lib.pg_kv_cache_free(B.h, kv)
        for h in hs:
            lib.pg_gguf_free(B.h, h)
    torch.cuda.empty_cache()


def section_huffman(B, line):
    """HuffmanTensor::to_gpu of a [4096 x 4096] int8 weight: host streams in, device tensor out."""
    import numpy as np

    lib, check = B.lib, B.check
    hk, hn, hstreams = 4096, 4096, 16
    hq = np.clip(np.rint(B.normal(7400, (hk * hn,), 9.0).cpu().numpy()), -24, 24).astype(np.int8)
    hscales = np.full(hn, 0.01, np.float32)
    ht = C.c_void_p()
    check(lib.pg_huffman_tensor_from_quantized(C.c_void_p(hq.ctypes.data), C.c_void_p(hscales.ctypes.data), hk, hn, hstreams,
                                               C.byref(ht)))
    hsz = C.c_size_t()
    check(lib.pg_huffman_tensor_info(ht, None, None, None, C.byref(hsz)))

    def huff_step():
        h = C.c_void_p()
        check(lib.pg_huffman_tensor_to_gpu(B.h, ht, C.byref(h)))
        lib.pg_qtensor_free(B.h, h)

    for _ in range(2):
        huff_step()
    t0 = time.perf_counter()
    for _ in range(5):
        huff_step()
    huff_ms = (time.perf_counter() - t0) / 5 * 1e3
    hprof, _ = B.profiled(huff_step, 5)
    huff_kernels_ms = sum(v[0] * v[1] for k, v in hprof.items() if k.startswith("huffman")) / 5
    line["huffman_to_gpu"] = {
        "workload": f"HuffmanTensor::to_gpu of a [{hk}x{hn}] int8 weight in {hstreams} streams "
                    f"({hsz.value / 1e6:.1f} MB compressed, ratio {(hk * hn + 4 * hn) / hsz.value:.2f}); host streams in, device tensor out",
        "ms_per_call_wall": round(huff_ms, 3), "decode_kernels_ms": round(huff_kernels_ms, 3),
        "symbols_per_s_kernels": round(hk * hn / (huff_kernels_ms * 1e-3), 0),
        "kernels_ms_x_launches": {k: [round(v[0], 4), round(v[1] / 5, 1)] for k, v in hprof.items()}}
    lib.pg_huffman_tensor_free(ht)


def section_huffman_kv(B, line):
    """HuffmanKVCache::compress_chunk / decompress_chunk on a chunk that is already on the device:
    8 KV heads x 256 tokens x 128 (1 MiB of f32 per side), wall time per call (each call waits for
    its histogram and for the stream's length, so kernel time is the smaller part)."""
    lib, check = B.lib, B.check
    heads, tokens, hd = 8, 256, 128
    n = heads * tokens * hd
    data = B.normal(7500, (n,), 1.0)
    out = B.torch.empty(n, dtype=B.torch.float32, device=data.device)
    chunk = C.c_void_p()

    def compress():
        h = C.c_void_p()
        check(lib.pg_huffman_kv_compress_chunk_dev(B.h, C.c_void_p(data.data_ptr()), tokens * hd, tokens, heads, hd, C.byref(h)))
        return h

    def comp_step():
        lib.pg_huffman_kv_chunk_free(B.h, compress())

    chunk = compress()
    nbytes = C.c_size_t()
    check(lib.pg_huffman_kv_chunk_info(chunk, None, None, None, C.byref(nbytes)))

    def dec_step():
        check(lib.pg_huffman_kv_decompress_chunk_dev(B.h, chunk, C.c_void_p(out.data_ptr()), tokens * hd))

    res = {}
    for name, fn in (("compress", comp_step), ("decompress", dec_step)):
        for _ in range(2):
            fn()
        B.torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            fn()
        B.torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / 10 * 1e3
        prof, _ = B.profiled(fn, 5)
        res[name] = {"ms_per_call_wall": round(wall, 3),
                     "kernels_ms": round(sum(v[0] * v[1] for v in prof.values()) / 5, 4),
                     "kernels_ms_x_launches": {k: [round(v[0], 4), round(v[1] / 5, 1)] for k, v in prof.items()}}
    # a cache of 8448 tokens: 32 chunks per side behind a window of 256 tokens; get_kv decodes all 64 streams in one pass
    cache = C.c_void_p()
    check(lib.pg_huffman_kv_cache_create(B.h, heads, hd, 2 * tokens, tokens, C.byref(cache)))
    piece = 1056
    kk, vv = B.normal(7501, (heads * piece * hd,), 1.0), B.normal(7502, (heads * piece * hd,), 2.0)
    B.torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(8):
        check(lib.pg_huffman_kv_cache_append_dev(B.h, cache, C.c_void_p(kk.data_ptr()), C.c_void_p(vv.data_ptr()), piece))
    B.torch.cuda.synchronize()
    append_ms = (time.perf_counter() - t0) / 8 * 1e3
    total_len, comp_len = lib.pg_huffman_kv_cache_len(cache), lib.pg_huffman_kv_cache_compressed_len(cache)
    full_k = B.torch.empty(heads * total_len * hd, dtype=B.torch.float32, device=data.device)
    full_v = B.torch.empty_like(full_k)

    def get_step():
        check(lib.pg_huffman_kv_cache_get_kv_dev(B.h, cache, C.c_void_p(full_k.data_ptr()), C.c_void_p(full_v.data_ptr())))

    for _ in range(2):
        get_step()
    B.torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        get_step()
    B.torch.cuda.synchronize()
    get_ms = (time.perf_counter() - t0) / 5 * 1e3
    gprof, _ = B.profiled(get_step, 3)
    res["cache"] = {"workload": f"{total_len} tokens ({comp_len} in {lib.pg_huffman_kv_cache_num_chunks(cache)} chunks per side), appended {piece} at a time from device tensors",
                    "append_ms_per_call_wall": round(append_ms, 3), "get_kv_dev_ms_wall": round(get_ms, 3),
                    "get_kv_dev_gbs_of_f32_out": round(2 * 4 * heads * total_len * hd / (get_ms * 1e-3) / 1e9, 1),
                    "get_kv_kernels_ms_x_launches": {k: [round(v[0], 4), round(v[1] / 3, 1)] for k, v in gprof.items()}}
    lib.pg_huffman_kv_cache_free(B.h, cache)
    del full_k, full_v, kk, vv
    if B.cpu:  # the scalar restatement of compress_chunk / decompress_chunk on the same chunk (the prebuilt -O2 oracle)
        import numpy as np
        olib = C.CDLL(os.path.join(ROOT, "oracle", "_build", "libperegrine_oracle.so"))
        olib.orc_huffman_kv_compress_chunk.restype = C.c_size_t
        host = data.cpu().numpy()
        bits, scales, book, back = np.zeros(2 * n + 16, np.uint8), np.zeros(heads, np.float32), np.zeros(256, np.uint8), np.zeros(n, np.float32)
        vp = lambda a: C.c_void_p(a.ctypes.data)
        sz = C.c_size_t
        best = [1e9, 1e9]
        for _ in range(3):
            t0 = time.perf_counter()
            nb = olib.orc_huffman_kv_compress_chunk(vp(host), sz(tokens), sz(heads), sz(hd), vp(bits), vp(scales), vp(book), None)
            t1 = time.perf_counter()
            olib.orc_huffman_kv_decompress_chunk(vp(bits), sz(nb), vp(scales), vp(book), sz(tokens), sz(heads), sz(hd), vp(back))
            best = [min(best[0], t1 - t0), min(best[1], time.perf_counter() - t1)]
        res["cpu_baseline"] = {"compress_ms": round(best[0] * 1e3, 3), "decompress_ms": round(best[1] * 1e3, 3), "cores": 1, "kind": "port",
                               "sample": "the same chunk, best of 3, single thread, gcc -O2"}
    line["huffman_kv_chunk"] = {
        "workload": f"HuffmanKVCache chunk of {heads} heads x {tokens} tokens x {hd} f32 on the device "
                    f"({4 * n / 1e6:.2f} MB -> {nbytes.value / 1e6:.3f} MB, {8 * nbytes.value / n:.2f} bits per value)",
        **res}
    lib.pg_huffman_kv_chunk_free(B.h, chunk)


# ---------------------------------------------------------------------- CPU baseline legs (the oracle; reported only)
CPU_ROWS = 512  # activation rows of the headline step the CPU leg runs (about 4 s on one core)


def load_oracle():
    """The scalar CPU oracle (the restatement of the reference's x86 path) as a host-tuned build:
    gcc -O3 -march=native; falls back to the prebuilt -O2 library."""
    src = os.path.join(ROOT, "oracle", "peregrine_oracle.c")
    so = os.path.join(ROOT, "oracle", "_build", "libperegrine_oracle.so")
    flags = "-O2, prebuilt"
    try:
        tmp = os.path.join(tempfile.mkdtemp(prefix="pg_cpu_"), "liboracle_native.so")
        subprocess.check_call(["gcc", "-O3", "-march=native", "-std=c11", "-fPIC", "-ffp-contract=off",
                               "-shared", "-o", tmp, src, "-lm"], stderr=subprocess.DEVNULL)
        so, flags = tmp, "-O3 -march=native"
    except Exception:
        pass
    lib = C.CDLL(so)
    lib.orc_dequant_q4_0.restype = C.c_int
    return {"lib": lib, "flags": flags}


def _best_of(fn, reps):
    best = None
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best = dt if best is None or dt < best else best
    return best


def _vp(a):
    return C.c_void_p(a.ctypes.data)


def cpu_baseline(orc, cpu_w, cpu_a):
    """The headline workload on one host core: a bounded sample of the step (CPU_ROWS of the 2048
    activation rows through all 7 products); the work is linear in the rows."""
    import numpy as np

    lib = orc["lib"]
    t_total, ops = 0.0, 0
    for name, k, n in LAYER:
        qt, sc = cpu_w[name]
        a = np.ascontiguousarray(cpu_a[k][:CPU_ROWS])
        out = np.empty(CPU_ROWS * n, np.float32)
        t0 = time.perf_counter()
        lib.orc_matmul_quantized(_vp(a), C.c_size_t(CPU_ROWS), C.c_size_t(k), _vp(qt), _vp(sc), C.c_size_t(n), _vp(out), None)
        t_total += time.perf_counter() - t0
        ops += 2 * CPU_ROWS * k * n
    return {"value": round(ops / t_total / 1e12, 5), "unit": "TOP/s", "cores": 1, "kind": "port",
            "sample": f"{CPU_ROWS} of {M_PREFILL} activation rows through all 7 products "
                      f"({ops / 2e9:.1f} G MAC in {t_total:.1f} s, single thread, gcc {orc['flags']}); "
                      "rate is per-row linear so it stands for the full step",
            "host_cores_available": os.cpu_count()}


def _cpu_quantize(lib, w_f32):
    import numpy as np

    k, n = w_f32.shape
    q, q_t, s = np.empty(k * n, np.int8), np.empty(k * n, np.int8), np.empty(n, np.float32)
    w = np.ascontiguousarray(w_f32, np.float32)
    lib.orc_quantize_weights(_vp(w), C.c_size_t(k), C.c_size_t(n), _vp(q), _vp(q_t), _vp(s))
    return q_t, s


def cpu_linear(orc, w_f32, a):
    """cfg1 at full size: quantize_weights once (untimed, a load-time step), then matmul_quantized."""
    import numpy as np

    lib = orc["lib"]
    k, n = w_f32.shape
    m = a.shape[0]
    q_t, s = _cpu_quantize(lib, w_f32)
    a = np.ascontiguousarray(a, np.float32)
    out = np.empty(m * n, np.float32)

    def run():
        lib.orc_matmul_quantized(_vp(a), C.c_size_t(m), C.c_size_t(k), _vp(q_t), _vp(s), C.c_size_t(n), _vp(out), None)

    dt = _best_of(run, 3)
    return {"value": round(2 * m * k * n / dt / 1e12, 5), "unit": "TOP/s", "ms": round(dt * 1e3, 2), "cores": 1, "kind": "port",
            "sample": f"the whole [{m}x{k}] x [{k}x{n}] product, best of 3, single thread, gcc {orc['flags']}"}


def cpu_decode(orc, kept, x_d, x_f, dec_bytes):
    """cfg2 at full size: the three M = 1 products of one layer through matmul_quantized."""
    import numpy as np

    lib = orc["lib"]
    prods = []
    for w_f32, x in zip(kept, (x_d, x_d, x_f)):
        k, n = w_f32.shape
        q_t, s = _cpu_quantize(lib, w_f32)
        prods.append((np.ascontiguousarray(x, np.float32).reshape(-1), k, n, q_t, s, np.empty(n, np.float32)))

    def run():
        for x, k, n, q_t, s, out in prods:
            lib.orc_matmul_quantized(_vp(x), C.c_size_t(1), C.c_size_t(k), _vp(q_t), _vp(s), C.c_size_t(n), _vp(out), None)

    dt = _best_of(run, 5)
    return {"value": round(dec_bytes / dt / 1e9, 2), "unit": "GB/s", "ms": round(dt * 1e3, 2), "cores": 1, "kind": "port",
            "sample": f"the whole step (three M=1 products, 176 M MAC), best of 5, single thread, gcc {orc['flags']}"}


def cpu_gguf(orc, raw, n_out, k_in, ms):
    """cfg4 at full size, as the reference composes it: dequantise the tensor to f32 and
    transpose it to [in, out] once (load time, src/models/llama/model.rs:243-257; not in the
    figure, its duration is stated), then Tensor::matmul's i-j-p loop per call."""
    import numpy as np

    lib = orc["lib"]
    wf = np.empty(n_out * k_in, np.float32)
    t0 = time.perf_counter()
    rc = lib.orc_dequant_q4_0(_vp(raw), C.c_size_t(n_out * k_in), _vp(wf))
    t_deq = time.perf_counter() - t0
    assert rc == 0
    w_t = np.ascontiguousarray(wf.reshape(n_out, k_in).T)  # [k_in, n_out]
    del wf
    res = {}
    rng = np.random.default_rng(3)
    for m in ms:
        x = rng.standard_normal((m, k_in)).astype(np.float32)
        y = np.empty(m * n_out, np.float32)

        def run():
            lib.orc_matmul_f32(_vp(x), _vp(w_t), C.c_size_t(m), C.c_size_t(k_in), C.c_size_t(n_out), _vp(y))

        dt = _best_of(run, 2 if m < 16 else 1)
        bytes_alg = n_out * (k_in // 32) * 18 + 4 * m * k_in + 4 * m * n_out
        res[m] = {"value": round(bytes_alg / dt / 1e9, 3), "unit": "GB/s", "ms": round(dt * 1e3, 1),
                  "gflops": round(2 * m * n_out * k_in / dt / 1e9, 2), "cores": 1, "kind": "port",
                  "sample": f"the whole [{m}x{k_in}] x [{k_in}x{n_out}] f32 product over the dequantised, transposed tensor "
                            f"(Tensor::matmul's i-j-p loop), single thread, gcc {orc['flags']}; the one-off dequantisation "
                            f"of the tensor took {t_deq * 1e3:.0f} ms and is not included"}
    return res


if __name__ == "__main__":
    main()
