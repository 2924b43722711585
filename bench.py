#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  Headline (`value`): W8A8 prefill GEMM throughput, in TOP/s, over the
seven projections of one Llama-3-8B layer at M = 2048 tokens (q, k, v, o, gate, up, down;
893 353 197 568 integer ops per step), each through `pg_matmul_quantized_dev` (per-row
activation quantisation + i8 MFMA GEMM + f32 rescale), inputs resident in HBM: two sets of
layer weights (436 MB, more than the Infinity Cache) are used alternately, and the step runs
untimed for 0.2 s before the W warm-up steps so that clocks and caches have settled.
The same line carries the decode leg of the metric (`decode_gemv`: M = 1 int8 GEMV GB/s at
the 8B FFN shapes, weights rotated through more distinct buffers than the 256 MB Infinity
Cache holds), the Q4_0 decode GEMV (`gguf_q4_0_gemv`), a `roofline` object per dominant
kernel (durations from HIP events recorded by the library on its own stream) and the CPU
baseline (`cpu_baseline`: the scalar oracle on this host's cores, one thread, bounded sample).

torch is used for device memory and for the whole-step timing events only.
"""
import argparse
import ctypes as C
import json
import os
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
    """profiles/hbm_traffic.json: per-kernel HBM bytes per launch derived from rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE runs of this benchmark, scaled by a plain copy of known size
    (the file names the commands).  Absent file -> traffic is reported as null."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            return json.load(f).get("bytes_per_launch", {})
    except (OSError, ValueError):
        return {}


TRAFFIC = load_traffic()


def gemv_bytes(k, n):
    """Algorithmic bytes of one M = 1 W8A8 product: i8 weights + w scales + f32 x + f32 out."""
    return k * n + 4 * n + 4 * k + 4 * n


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU baseline leg")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain 512 MiB device copies (counter calibration under rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; every kernel here runs at its real "
                 "single-GPU shape. Run with --gpus 1.")

    import numpy as np
    import torch
    from peregrine_amd import _ffi, Context

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; peregrine_amd has no CPU path to measure")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    # A dedicated (non-null) stream shared by torch and the library, so the torch events
    # that bracket the timed region see the library's kernels.
    stream = torch.cuda.Stream(device=dev)
    torch.cuda.set_stream(stream)
    assert stream.cuda_stream != 0
    ctx = Context(0, stream=stream.cuda_stream)
    assert ctx.stream == stream.cuda_stream
    lib, check = _ffi.lib, _ffi.check
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)

    def ptr(t):
        return C.c_void_p(t.data_ptr())

    def make_weight(k, n):
        w = torch.randn(k, n, device=dev, generator=gen, dtype=torch.float32) * 0.02
        h = C.c_void_p()
        check(lib.pg_qtensor_from_f32_dev(ctx.handle, ptr(w), k, n, C.byref(h)))
        del w
        return h

    def make_acts(m, k):
        a = torch.randn(m, k, device=dev, generator=gen, dtype=torch.float32)
        chan = torch.randperm(k, device=dev, generator=gen)[: max(1, k // 100)]
        a[:, chan] *= 20.0  # 1 % outlier channels
        return a.contiguous()

    def timed(fn, steps, warmup):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(steps):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps  # ms per step

    def profiled(fn, steps):
        """Per-kernel durations from the library's HIP events: each dispatch carries a start
        and a stop event stamped with the kernel's own begin/end on the stream it runs on
        (hipExtLaunchKernel), so the figures are comparable with a rocprofv3 kernel trace.
        Returns {name: (avg_ms, launches)}."""
        ctx.profile_begin()
        for _ in range(steps):
            fn()
        return {name: (total / n, n) for name, (total, n) in ctx.profile_end().items()}

    def traffic_for(kernel):
        """HBM bytes per launch from the committed rocprofv3 --pmc measurement, or None."""
        return TRAFFIC.get(kernel)

    # ------------------------------------------------------------------ prefill (headline)
    # Two layers' worth of weights (436 MB), used alternately: more than the 256 MB Infinity Cache
    # holds, so every step streams its weights from HBM as a model with many layers would
    # (with one set reused every step the layer runs about 3 % faster).
    weight_sets = [{name: make_weight(k, n) for name, k, n in LAYER} for _ in range(2)]
    weights = weight_sets[0]
    prefill_state = {"i": 0}
    acts = {4096: make_acts(M_PREFILL, 4096), 14336: make_acts(M_PREFILL, 14336)}
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
        ws = weight_sets[prefill_state["i"] % len(weight_sets)]
        prefill_state["i"] += 1
        a4, a14 = ptr(acts[4096]), ptr(acts[14336])
        check(lib.pg_matmul_quantized_multi_dev(ctx.handle, a4, M_PREFILL, 4096, ws["qkv_tab"], 3, qkv_out))
        check(lib.pg_matmul_quantized_dev(ctx.handle, a4, M_PREFILL, 4096, ws["o_proj"], ptr(outs[4096]), None))
        check(lib.pg_matmul_quantized_multi_dev(ctx.handle, a4, M_PREFILL, 4096, ws["gu_tab"], 2, gu_out))
        check(lib.pg_matmul_quantized_dev(ctx.handle, a14, M_PREFILL, 14336, ws["down_proj"], ptr(outs[4096]), None))

    # Clocks and caches need tens of milliseconds of this work to settle (a 3 ms warm-up leaves
    # the layer about 8 % slower than its steady state): run it untimed for SETTLE_S first, then
    # the W warm-up steps and the K timed ones as asked.
    t_settle = time.time()
    while time.time() - t_settle < SETTLE_S:
        for _ in range(10):
            prefill_step()
        torch.cuda.synchronize()
    ms_step = timed(prefill_step, args.steps, args.warmup)
    tops = LAYER_OPS / (ms_step * 1e-3) / 1e12
    prof = profiled(prefill_step, args.steps)
    gemm_avg_ms, g_n = prof["gemm_w8a8"]
    q_avg_ms, q_n = prof["quantize_rows"]
    gemm_lps = g_n / args.steps  # GEMM launches per step (a product may run as two column panels)
    gemm_tops = (LAYER_OPS / gemm_lps) / (gemm_avg_ms * 1e-3) / 1e12
    quant_ks = (4096, 4096, 4096, 14336)  # one quantisation per call of the step
    quant_bytes = sum(M_PREFILL * k * 4 + M_PREFILL * k + M_PREFILL * 4 for k in quant_ks)
    roofline = {"kernel": "gemm_w8a8_kernel (i8 MFMA 32x32x32; the 7 products as 4 launches: q|k|v, o, gate|up, down)", "bound": "mfma",
                "achieved": round(gemm_tops, 1), "peak": PEAK_INT8_TOPS, "unit": "TFLOP/s",
                "frac": round(gemm_tops / PEAK_INT8_TOPS, 4), "traffic": traffic_for("gemm_w8a8"),
                "ops_per_launch": int(LAYER_OPS / gemm_lps), "launches_per_step": gemm_lps, "avg_launch_ms": round(gemm_avg_ms, 4),
                "note": "unit counts int8 multiply-adds as 2 ops (TOP/s); duration from the HIP events "
                        "attached to each dispatch"}
    act_quant = {"kernel": "quantize_rows_vec4_kernel", "bound": "hbm",
                 "achieved": round(quant_bytes / len(quant_ks) / (q_avg_ms * 1e-3) / 1e9, 1),
                 "peak": PEAK_HBM_GBS, "unit": "GB/s", "avg_launch_ms": round(q_avg_ms, 4),
                 "traffic": traffic_for("quantize_rows")}
    act_quant["frac"] = round(act_quant["achieved"] / PEAK_HBM_GBS, 4)

    # Per product shape: this library's GEMM kernel beside the vendor library's int8 GEMM
    # (torch._int_mm = hipBLASLt; same operand layouts, i32 output without the rescale) on
    # random int8 operands.  A calibration of what int8 matrix-core code reaches on this
    # part at these sizes, not a figure of this library.
    vendor = []
    for name, k, n in (("q/o_proj", 4096, 4096), ("gate/up_proj", 4096, 14336), ("down_proj", 14336, 4096)):
        wname = {"q/o_proj": "q_proj", "gate/up_proj": "gate_proj", "down_proj": "down_proj"}[name]

        def one_product():
            check(lib.pg_matmul_quantized_dev(ctx.handle, ptr(acts[k]), M_PREFILL, k, weights[wname], ptr(outs[n]), None))

        for _ in range(3):
            one_product()
        ours_ms = profiled(one_product, 10)["gemm_w8a8"]
        ours_ms = ours_ms[0] * ours_ms[1] / 10  # per product (a product may run as two launches)
        entry = {"shape": f"{name}: [{M_PREFILL}x{k}] x [{k}x{n}]", "gemm_w8a8_ms": round(ours_ms, 4),
                 "gemm_w8a8_tops": round(2 * M_PREFILL * k * n / (ours_ms * 1e-3) / 1e12, 1)}
        try:
            va = torch.randint(-127, 128, (M_PREFILL, k), dtype=torch.int8, device=dev)
            vb = torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev).t()
            v_ms = timed(lambda: torch._int_mm(va, vb), 20, 5)
            entry["vendor_int_mm_ms"] = round(v_ms, 4)
            entry["vendor_int_mm_tops"] = round(2 * M_PREFILL * k * n / (v_ms * 1e-3) / 1e12, 1)
            del va, vb
        except Exception as exc:  # the calibration is optional
            entry["vendor_int_mm_error"] = repr(exc)[:120]
        vendor.append(entry)

    # ------------------------------------------------------------------ W8A32 (the reference's GPU numerics), gate product
    def w8a32_step():
        check(lib.pg_matmul_dequant_i8_dev(ctx.handle, ptr(acts[4096]), M_PREFILL, 4096, weights["gate_proj"], ptr(outs[14336])))

    w32_ms = timed(w8a32_step, args.steps, args.warmup)
    prof32 = profiled(w8a32_step, args.steps)
    w8a32 = {"workload": "W8A32 product [2048x4096] x [4096x14336] (f32 activations, dequantised i8 weights, f32 accumulate): "
                         "three int8 matrix-core passes over 24-bit fixed-point activations",
             "value": round(2 * M_PREFILL * 4096 * 14336 / (w32_ms * 1e-3) / 1e12, 1), "unit": "TFLOP/s",
             "ms_per_step": round(w32_ms, 4), "kernels_ms": {k: round(v[0], 5) for k, v in prof32.items()}}

    # keep one set of device-quantised weights on the host for the CPU baseline, then free
    cpu_w = {}
    if not args.skip_cpu:
        for name, k, n in LAYER:
            qt = np.empty(k * n, np.int8)
            sc = np.empty(n, np.float32)
            check(lib.pg_qtensor_download(ctx.handle, weights[name], None, C.c_void_p(qt.ctypes.data),
                                          C.c_void_p(sc.ctypes.data)))
            cpu_w[name] = (qt, sc)
        cpu_a = {k: acts[k].cpu().numpy().copy() for k in acts}
    for ws in weight_sets:
        for name, _, _ in LAYER:
            lib.pg_qtensor_free(ctx.handle, ws[name])
    del acts, outs
    torch.cuda.empty_cache()

    # ------------------------------------------------------------------ decode GEMV (int8)
    LAYERS_ROT = 4  # 4 x (gate, up, down) = 704 MB of distinct weights > 256 MB Infinity Cache
    dec_w = [(make_weight(4096, 14336), make_weight(4096, 14336), make_weight(14336, 4096))
             for _ in range(LAYERS_ROT)]
    x_d, x_f = make_acts(1, 4096), make_acts(1, 14336)
    y_f, y_d = torch.empty(1, 14336, device=dev), torch.empty(1, 4096, device=dev)
    state = {"i": 0}

    def decode_step():
        g, u, d = dec_w[state["i"] % LAYERS_ROT]
        state["i"] += 1
        check(lib.pg_matmul_quantized_dev(ctx.handle, ptr(x_d), 1, 4096, g, ptr(y_f), None))
        check(lib.pg_matmul_quantized_dev(ctx.handle, ptr(x_d), 1, 4096, u, ptr(y_f), None))
        check(lib.pg_matmul_quantized_dev(ctx.handle, ptr(x_f), 1, 14336, d, ptr(y_d), None))

    dec_bytes = 2 * gemv_bytes(4096, 14336) + gemv_bytes(14336, 4096)
    dsteps = max(args.steps * 10, 100)
    dec_ms = timed(decode_step, dsteps, max(args.warmup, 8))
    prof = profiled(decode_step, dsteps)
    gemv_avg_ms, v_n = prof["gemv_w8a8"]
    gemv_gbs = (dec_bytes / 3) / (gemv_avg_ms * 1e-3) / 1e9
    decode = {"workload": "cfg2: M=1 int8 GEMV, x[4096]->gate,up[14336], x[14336]->down[4096]; "
                          f"{LAYERS_ROT} layers of weights rotated ({LAYERS_ROT * 3 * 58.7:.0f} MB, HBM-resident reads)",
              "value": round(dec_bytes / (dec_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
              "ms_per_step": round(dec_ms, 5), "steps": dsteps, "bytes_per_step": dec_bytes,
              "roofline": {"kernel": "gemv_w8a8_m1_f32x_kernel (quantises its activation row, then streams the weights)", "bound": "hbm", "achieved": round(gemv_gbs, 1),
                           "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gemv_gbs / PEAK_HBM_GBS, 4),
                           "traffic": traffic_for("gemv_w8a8"), "bytes_per_launch": dec_bytes // 3,
                           "avg_launch_ms": round(gemv_avg_ms, 5)}}
    for trio in dec_w:
        for h in trio:
            lib.pg_qtensor_free(ctx.handle, h)
    torch.cuda.empty_cache()

    # ------------------------------------------------------------------ cfg1: one W8A8 linear, M = 32
    w1 = [make_weight(4096, 4096) for _ in range(8)]  # 8 x 16.8 MB rotated
    a1 = torch.randn(32, 4096, device=dev, generator=gen, dtype=torch.float32)
    o1 = torch.empty(32, 4096, device=dev)

    def lin_step():
        h = w1[state["i"] % len(w1)]
        state["i"] += 1
        check(lib.pg_matmul_quantized_dev(ctx.handle, ptr(a1), 32, 4096, h, ptr(o1), None))

    lin_ms = timed(lin_step, dsteps, max(args.warmup, 8))
    prof = profiled(lin_step, dsteps)
    lin_bytes = 17842176
    linear_m32 = {"workload": "cfg1: W8A8 linear [32x4096] x [4096x4096] (the reference's CPU-runnable case); 8 weights rotated",
                  "value": round(2 * 32 * 4096 * 4096 / (lin_ms * 1e-3) / 1e12, 2), "unit": "TOP/s",
                  "gbs": round(lin_bytes / (lin_ms * 1e-3) / 1e9, 1), "ms_per_step": round(lin_ms, 5),
                  "kernels_ms": {k: round(v[0], 5) for k, v in prof.items()}}
    for h in w1:
        lib.pg_qtensor_free(ctx.handle, h)

    # ------------------------------------------------------------------ decode GEMV (GGUF Q4_0)
    from peregrine_amd import synth
    n_out, k_in = 14336, 4096
    wq = (torch.randn(n_out, k_in, generator=torch.Generator().manual_seed(7)) * 0.02).numpy()
    raw = np.frombuffer(synth.pack_q4_0(wq), np.uint8)
    Q4_ROT = 10  # 10 x 33 MB = 330 MB of distinct Q4_0 tensors
    q4 = []
    for _ in range(Q4_ROT):
        h = C.c_void_p()
        check(lib.pg_gguf_upload(ctx.handle, C.c_void_p(raw.ctypes.data), _ffi.GGML_Q4_0, n_out, k_in, C.byref(h)))
        q4.append(h)
    y_q = torch.empty(1, n_out, device=dev)

    def q4_step():
        h = q4[state["i"] % Q4_ROT]
        state["i"] += 1
        check(lib.pg_gguf_matmul_dev(ctx.handle, ptr(x_d), 1, h, ptr(y_q)))

    q4_bytes = n_out * (k_in // 32) * 18 + 4 * k_in + 4 * n_out  # 33 103 872
    q4_ms = timed(q4_step, dsteps, max(args.warmup, 8))
    prof = profiled(q4_step, dsteps)
    q4_avg_ms, k_n = prof["gguf_gemv_q4_0"]
    q4_gbs = q4_bytes / (q4_avg_ms * 1e-3) / 1e9
    gguf = {"workload": f"cfg4: M=1 Q4_0 dequant-GEMV [4096]->[14336]; {Q4_ROT} tensors rotated (330 MB)",
            "value": round(q4_bytes / (q4_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "ms_per_step": round(q4_ms, 5),
            "roofline": {"kernel": "gguf_gemv_kernel<Q4_0>", "bound": "hbm", "achieved": round(q4_gbs, 1),
                         "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(q4_gbs / PEAK_HBM_GBS, 4),
                         "traffic": traffic_for("gguf_gemv_q4_0"), "bytes_per_launch": q4_bytes,
                         "avg_launch_ms": round(q4_avg_ms, 5)}}
    # ------------------------------------------------------------------ cfg4 at M = 4 and 16 (matrix-core path)
    skinny = []
    for m_q in (4, 16):
        x_m = torch.randn(m_q, k_in, device=dev, generator=gen, dtype=torch.float32)
        y_m = torch.empty(m_q, n_out, device=dev)

        def mm_step():
            h = q4[state["i"] % Q4_ROT]
            state["i"] += 1
            check(lib.pg_gguf_matmul_dev(ctx.handle, ptr(x_m), m_q, h, ptr(y_m)))

        mm_bytes = n_out * (k_in // 32) * 18 + 4 * m_q * k_in + 4 * m_q * n_out
        mm_ms = timed(mm_step, dsteps, max(args.warmup, 8))
        prof = profiled(mm_step, dsteps)
        k_ms = prof["gguf_mm_q4_0"][0]
        skinny.append({"workload": f"cfg4: M={m_q} Q4_0 dequant-matmul [{m_q}x4096]->[{m_q}x14336], weights read once",
                       "value": round(mm_bytes / (mm_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "ms_per_step": round(mm_ms, 5),
                       "gflops": round(2 * m_q * n_out * k_in / (mm_ms * 1e-3) / 1e9, 1),
                       "kernels_ms": {k: round(v[0], 5) for k, v in prof.items()},
                       "roofline": {"kernel": "gguf_mm_kernel<Q4_0>", "bound": "hbm",
                                    "achieved": round(mm_bytes / (k_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                    "frac": round(mm_bytes / (k_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": traffic_for("gguf_mm_q4_0"),
                                    "bytes_per_launch": mm_bytes, "avg_launch_ms": round(k_ms, 5)}})
    for h in q4:
        lib.pg_gguf_free(ctx.handle, h)
    del raw, wq

    # ------------------------------------------------------------------ cfg5: Grok-1-shaped MoE expert FFN, Q8_0
    T_moe, d_moe, ffn_moe, E_moe, topk_moe = 64, 6144, 32768, 8, 2
    nblk = ffn_moe * d_moe // 32
    rng = np.random.default_rng(5)
    blocks = np.empty((nblk, 34), np.uint8)
    blocks[:, 2:] = rng.integers(0, 256, size=(nblk, 32), dtype=np.uint8)      # i8 quants
    blocks[:, :2] = np.frombuffer(np.float16(0.02 / 127).tobytes(), np.uint8)  # d
    experts = [[], [], []]
    for which, (no, ki) in enumerate(((ffn_moe, d_moe), (ffn_moe, d_moe), (d_moe, ffn_moe))):
        for e in range(E_moe):
            blocks[:, 2] = e + 8 * which  # make the tensors differ
            h = C.c_void_p()
            check(lib.pg_gguf_upload(ctx.handle, C.c_void_p(blocks.ctypes.data), _ffi.GGML_Q8_0, no, ki, C.byref(h)))
            experts[which].append(h)
    del blocks
    tabs = [(C.c_void_p * E_moe)(*[h.value for h in experts[w]]) for w in range(3)]
    x_moe = torch.randn(T_moe, d_moe, device=dev, generator=gen, dtype=torch.float32)
    lg_moe = torch.randn(T_moe, E_moe, device=dev, generator=gen, dtype=torch.float32)
    out_moe = torch.empty(T_moe, d_moe, device=dev)

    def moe_step():
        check(lib.pg_moe_ffn_dev(ctx.handle, ptr(x_moe), T_moe, ptr(lg_moe), E_moe, topk_moe, tabs[0], tabs[1], tabs[2],
                                 _ffi.ACT_SILU, ptr(out_moe)))

    moe_bytes = 3 * E_moe * nblk * 34 + 2 * 4 * T_moe * d_moe  # every expert is hit at T=64, k=2 (checked below)
    hit = int(torch.unique(torch.topk(lg_moe, topk_moe, dim=1).indices).numel())
    moe_ms = timed(moe_step, 20, 10)  # 5 GB of weights: the first passes also warm the TLBs
    prof = profiled(moe_step, 5)
    mm_total = prof["gguf_mm_q8_0"][0] * prof["gguf_mm_q8_0"][1] / 5  # three launches per step
    moe = {"workload": "cfg5: Grok-1-shaped MoE FFN, Q8_0 experts (d 6144, ffn 32768, 8 experts, top-2, 64 tokens, SiLU); "
                       "5.13 GB of expert weights, read once per step",
           "experts_hit": hit, "value": round(moe_bytes / (moe_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
           "ms_per_step": round(moe_ms, 4),
           "tflops": round(2 * T_moe * topk_moe * 3 * ffn_moe * d_moe / (moe_ms * 1e-3) / 1e12, 2),
           "kernels_ms": {k: round(v[0], 5) for k, v in prof.items()},
           "roofline": {"kernel": "gguf_mm_kernel<Q8_0> (gate, up, down)", "bound": "hbm",
                        "achieved": round(3 * E_moe * nblk * 34 / (mm_total * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                        "unit": "GB/s", "frac": round(3 * E_moe * nblk * 34 / (mm_total * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                        "traffic": traffic_for("gguf_mm_q8_0"), "bytes_per_launch": E_moe * nblk * 34,
                        "avg_launch_ms": round(prof["gguf_mm_q8_0"][0], 5)}}
    for w3 in experts:
        for h in w3:
            lib.pg_gguf_free(ctx.handle, h)
    torch.cuda.empty_cache()

    # ------------------------------------------------------------------ one Llama-3-8B decoder block, Q4_0 weights
    d_l, nqh_l, nkv_l, hd_l, ffn_l, ctx_len = 4096, 32, 8, 128, 14336, 1024
    shapes_l = [(nqh_l * hd_l, d_l), (nkv_l * hd_l, d_l), (nkv_l * hd_l, d_l), (d_l, nqh_l * hd_l),
                (ffn_l, d_l), (ffn_l, d_l), (d_l, ffn_l)]
    L_ROT = 4  # 4 x 123 MB of block weights rotated: more than the 256 MB last-level cache
    rng = np.random.default_rng(8)
    blocks_l, keep_l = [], []
    for r in range(L_ROT):
        hs = []
        for no, ki in shapes_l:
            nb = no * ki // 32
            rawb = np.empty((nb, 18), np.uint8)
            rawb[:, 2:] = rng.integers(0, 256, size=(nb, 16), dtype=np.uint8)
            rawb[:, :2] = np.frombuffer(np.float16(0.02 / 7 * 64 / np.sqrt(ki)).tobytes(), np.uint8)
            h = C.c_void_p()
            check(lib.pg_gguf_upload(ctx.handle, C.c_void_p(rawb.ctypes.data), _ffi.GGML_Q4_0, no, ki, C.byref(h)))
            hs.append(h)
        b = C.c_void_p()
        check(lib.pg_llama_block_create(ctx.handle, d_l, nqh_l, nkv_l, hd_l, ffn_l, 4096, 500000.0, 1e-5, C.byref(b)))
        ones = np.ones(d_l, np.float32)
        check(lib.pg_llama_block_set_weights(ctx.handle, b, *hs, C.c_void_p(ones.ctypes.data), C.c_void_p(ones.ctypes.data)))
        kv = C.c_void_p()
        check(lib.pg_kv_cache_create(ctx.handle, nkv_l, hd_l, C.byref(kv)))
        blocks_l.append((b, kv))
        keep_l.append(hs)
    w_bytes_l = sum(no * ki // 32 * 18 for no, ki in shapes_l)
    h_pre = torch.randn(ctx_len, d_l, device=dev, generator=gen, dtype=torch.float32)
    o_pre = torch.empty_like(h_pre)
    h_dec = torch.randn(1, d_l, device=dev, generator=gen, dtype=torch.float32)
    o_dec = torch.empty_like(h_dec)

    def block_prefill():
        b, kv = blocks_l[state["i"] % L_ROT]
        state["i"] += 1
        check(lib.pg_kv_cache_rollback_to(kv, 0))
        check(lib.pg_llama_block_forward_dev(ctx.handle, b, ptr(h_pre), ctx_len, kv, ptr(o_pre)))

    def block_decode():  # position ctx_len on top of the prefilled cache, then rolled back
        b, kv = blocks_l[state["i"] % L_ROT]
        state["i"] += 1
        check(lib.pg_kv_cache_rollback_to(kv, ctx_len))
        check(lib.pg_llama_block_forward_dev(ctx.handle, b, ptr(h_dec), 1, kv, ptr(o_dec)))

    pre_ms = timed(block_prefill, 16, 8)  # leaves every cache filled to ctx_len
    pre_prof = profiled(block_prefill, 8)
    dec_ms = timed(block_decode, dsteps, max(args.warmup, 8))
    dec_prof = profiled(block_decode, dsteps)
    kv_bytes_l = 2 * nkv_l * (ctx_len + 1) * hd_l * 4
    dec_bytes = w_bytes_l + kv_bytes_l
    pre_flops = 2 * ctx_len * sum(no * ki for no, ki in shapes_l) + 4 * nqh_l * hd_l * ctx_len * (ctx_len + 1) // 2
    llama_block = {
        "workload": f"one Llama-3-8B decoder block (d 4096, 32/8 heads x 128, ffn 14336), Q4_0 projections ({w_bytes_l / 1e6:.0f} MB), "
                    f"f32 KV cache; {L_ROT} blocks rotated",
        "decode": {"what": f"seq 1 at position {ctx_len}", "ms_per_step": round(dec_ms, 5),
                   "value": round(dec_bytes / (dec_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                   "frac_of_hbm_peak": round(dec_bytes / (dec_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                   "bytes_per_step": dec_bytes,
                   "kernels_ms_x_launches": {k: [round(v[0], 5), round(v[1] / dsteps, 2)] for k, v in dec_prof.items()}},
        "prefill": {"what": f"seq {ctx_len} into an empty cache", "ms_per_step": round(pre_ms, 4),
                    "tflops": round(pre_flops / (pre_ms * 1e-3) / 1e12, 1),
                    "tokens_per_s": round(ctx_len / (pre_ms * 1e-3), 0),
                    "kernels_ms_x_launches": {k: [round(v[0], 5), round(v[1] / 8, 2)] for k, v in pre_prof.items()}},
    }
    for (b, kv), hs in zip(blocks_l, keep_l):
        lib.pg_llama_block_free(ctx.handle, b)
        lib.pg_kv_cache_free(ctx.handle, kv)
        for h in hs:
            lib.pg_gguf_free(ctx.handle, h)
    torch.cuda.empty_cache()

    # ------------------------------------------------------------------ Huffman-coded weight -> device tensor
    hk, hn, hstreams = 4096, 4096, 16
    hq = np.clip(np.rint(np.random.default_rng(21).standard_normal(hk * hn) * 9.0), -24, 24).astype(np.int8)
    hscales = np.full(hn, 0.01, np.float32)
    ht = C.c_void_p()
    check(lib.pg_huffman_tensor_from_quantized(C.c_void_p(hq.ctypes.data), C.c_void_p(hscales.ctypes.data), hk, hn, hstreams,
                                               C.byref(ht)))
    hsz = C.c_size_t()
    check(lib.pg_huffman_tensor_info(ht, None, None, None, C.byref(hsz)))

    def huff_step():
        h = C.c_void_p()
        check(lib.pg_huffman_tensor_to_gpu(ctx.handle, ht, C.byref(h)))
        lib.pg_qtensor_free(ctx.handle, h)

    for _ in range(2):
        huff_step()
    t0 = time.perf_counter()
    for _ in range(5):
        huff_step()
    huff_ms = (time.perf_counter() - t0) / 5 * 1e3
    hprof = profiled(huff_step, 5)
    huff_kernels_ms = sum(v[0] * v[1] for k, v in hprof.items() if k.startswith("huffman")) / 5
    huffman = {"workload": f"HuffmanTensor::to_gpu of a [{hk}x{hn}] int8 weight in {hstreams} streams "
                           f"({hsz.value / 1e6:.1f} MB compressed, ratio {(hk * hn + 4 * hn) / hsz.value:.2f}); host streams in, device tensor out",
               "ms_per_call_wall": round(huff_ms, 3), "decode_kernels_ms": round(huff_kernels_ms, 3),
               "symbols_per_s_kernels": round(hk * hn / (huff_kernels_ms * 1e-3), 0),
               "kernels_ms_x_launches": {k: [round(v[0], 4), round(v[1] / 5, 1)] for k, v in hprof.items()}}
    lib.pg_huffman_tensor_free(ht)
    del hq

    if args.calibrate_copy:  # a plain copy of known size: 512 MiB read + 512 MiB written per launch
        src = torch.empty(128 << 20, device=dev, dtype=torch.float32).normal_()
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ------------------------------------------------------------------ CPU baseline (oracle)
    cpu = None
    if not args.skip_cpu:
        cpu = cpu_baseline(cpu_w, cpu_a)

    line = {
        "metric": METRIC, "value": round(tops, 2), "unit": "TOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "cfg3: W8A8 prefill GEMMs of one Llama-3-8B layer at M=2048 "
                               "(q 4096->4096, k/v 4096->1024, o 4096->4096, gate/up 4096->14336, down 14336->4096), "
                               "activations N(0,1) with 1% channels x20, weights N(0,0.02), two weight sets (436 MB) alternated so that they stream from HBM, "
                               "each product = per-row activation quantisation + i8 GEMM + f32 rescale",
                   "m": M_PREFILL, "ops_per_step": LAYER_OPS, "untimed_settle_s": SETTLE_S},
        "pct_int8_mfma_peak": round(100 * tops / PEAK_INT8_TOPS, 2),
        "roofline": roofline, "gemm_vs_vendor_library": vendor, "activation_quant": act_quant, "w8a32_gate": w8a32, "linear_m32": linear_m32, "decode_gemv": decode, "gguf_q4_0_gemv": gguf, "gguf_q4_0_skinny": skinny, "moe_q8_0": moe, "llama_block_q4_0": llama_block, "huffman_to_gpu": huffman,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line), flush=True)
    ctx.close()


def cpu_baseline(cpu_w, cpu_a):
    """Time the scalar CPU oracle (the restatement of the reference's x86 path) on a bounded
    sample of the headline workload: one full step (all 2048 activation rows through all 7 products), about 15 s."""
    import numpy as np

    src = os.path.join(ROOT, "oracle", "peregrine_oracle.c")
    so = os.path.join(ROOT, "oracle", "_build", "libperegrine_oracle.so")
    flags = "-O2, prebuilt"
    try:  # a host-tuned build, as the measurement plan asks; fall back to the prebuilt one
        tmp = os.path.join(tempfile.mkdtemp(prefix="pg_cpu_"), "liboracle_native.so")
        subprocess.check_call(["gcc", "-O3", "-march=native", "-std=c11", "-fPIC", "-ffp-contract=off",
                               "-shared", "-o", tmp, src, "-lm"], stderr=subprocess.DEVNULL)
        so, flags = tmp, "-O3 -march=native"
    except Exception:
        pass
    lib = C.CDLL(so)
    rows = 2048  # the whole step: about 15 s of scalar CPU work
    t_total, ops = 0.0, 0
    for name, k, n in LAYER:
        qt, sc = cpu_w[name]
        a = np.ascontiguousarray(cpu_a[k][:rows])
        out = np.empty(rows * n, np.float32)
        t0 = time.perf_counter()
        lib.orc_matmul_quantized(C.c_void_p(a.ctypes.data), C.c_size_t(rows), C.c_size_t(k),
                                 C.c_void_p(qt.ctypes.data), C.c_void_p(sc.ctypes.data), C.c_size_t(n),
                                 C.c_void_p(out.ctypes.data), None)
        t_total += time.perf_counter() - t0
        ops += 2 * rows * k * n
    return {"value": round(ops / t_total / 1e12, 5), "unit": "TOP/s", "cores": 1, "kind": "port",
            "sample": f"{rows} of {M_PREFILL} activation rows through all 7 products "
                      f"({ops / 2e9:.1f} G MAC in {t_total:.1f} s, single thread, gcc {flags}); "
                      "rate is per-row linear so it stands for the full step",
            "host_cores_available": os.cpu_count()}


if __name__ == "__main__":
    main()
