"""The block step under stream capture: pg_llama_block_forward_dev, once its buffers exist, only launches
kernels on the context's stream, so a caller may capture a step into a hipGraph and replay it.

A replay must give what the eager step gives, every time: each graph is replayed several times with eager
work of the library on the same stream in between, and each replay is compared bit for bit with the eager
result for the input the buffer holds at that moment (the graph reads its input where the eager call did)."""
import ctypes as C
import sys

import numpy as np
import pytest

import helpers as H
from devbuf import DevBuf

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


class Hip:
    """The four runtime calls a capture needs, from the HIP runtime the library itself is linked with."""

    def __init__(self):
        # the copy of the runtime that is already mapped into this process (torch's, which the library bound to): a bare
        # name could resolve to another file and put a second runtime beside it
        path = "libamdhip64.so"
        with open("/proc/self/maps") as maps:
            for line in maps:
                if "libamdhip64" in line:
                    path = line.split()[-1]
                    break
        self.lib = C.CDLL(path)
        for name, args in (("hipStreamBeginCapture", [C.c_void_p, C.c_int]), ("hipStreamEndCapture", [C.c_void_p, C.POINTER(C.c_void_p)]),
                           ("hipGraphInstantiate", [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
                           ("hipGraphLaunch", [C.c_void_p, C.c_void_p]), ("hipGraphExecDestroy", [C.c_void_p]),
                           ("hipGraphDestroy", [C.c_void_p]), ("hipStreamSynchronize", [C.c_void_p])):
            fn = getattr(self.lib, name)
            fn.argtypes, fn.restype = args, C.c_int

    def ok(self, rc, what):
        assert rc == 0, f"{what}: hipError {rc}"

    def capture(self, stream, fn):
        graph, ex = C.c_void_p(), C.c_void_p()
        self.ok(self.lib.hipStreamBeginCapture(stream, 1), "hipStreamBeginCapture")   # thread-local: a forbidden call fails the capture
        try:
            fn()
        finally:
            rc = self.lib.hipStreamEndCapture(stream, C.byref(graph))
        self.ok(rc, "hipStreamEndCapture")
        self.ok(self.lib.hipGraphInstantiate(C.byref(ex), graph, None, None, 0), "hipGraphInstantiate")
        return graph, ex


@pytest.mark.parametrize("typ,seq,f16_route", [(2, 1, False), (8, 1, False), (2, 4, False), (2, 40, True), (8, 40, True)])
def test_block_step_replayed_from_a_graph(ctx, orc, typ, seq, f16_route):
    """f16_route: a many-token step with its products forced onto the f16 matrix cores (planes written by RMSNorm and
    SiLU.up, K chunks summed by the consumers): what a captured prefill chunk of a large model runs."""
    from peregrine_amd import _ffi
    if f16_route:
        _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 1))
    try:
        _block_step_replayed(ctx, orc, typ, seq)
    finally:
        _ffi.check(_ffi.lib.pg_gguf_hmm_force(ctx.handle, 0))


def _block_step_replayed(ctx, orc, typ, seq):
    from peregrine_amd import _ffi, gguf, llama
    hip = Hip()
    d, nqh, nkvh, hd, ffn, pre = 256, 8, 2, 64, 512, 300     # 300 positions: the keys are cut into splits / runs
    shapes = [(nqh * hd, d), (nkvh * hd, d), (nkvh * hd, d), (d, nqh * hd), (ffn, d), (ffn, d), (d, ffn)]
    pack = {2: H.pack_q4_0, 8: H.pack_q8_0}[typ]
    ws = [gguf.GgufWeight(bytes(pack(orc.rng_normal(70 + i, n * k, 0.0, 1.0 / np.sqrt(k)))), typ, n, k, ctx)
          for i, (n, k) in enumerate(shapes)]
    blk = llama.LlamaBlock(d, nqh, nkvh, hd, ffn, 512, 10000.0, 1e-5, ctx)
    blk.set_weights(*ws, (1 + 0.1 * orc.rng_normal(1, d)).astype(np.float32), (1 + 0.1 * orc.rng_normal(2, d)).astype(np.float32))
    cache = blk.new_cache()
    blk.forward(orc.rng_normal(3, pre * d).reshape(pre, d), cache)
    inputs = [orc.rng_normal(10 + i, seq * d) for i in range(4)]
    h_dev, o_dev = DevBuf(ctx, host=inputs[0]), DevBuf(ctx, seq * d * 4)
    other_in, other_out = DevBuf(ctx, host=orc.rng_normal(20, 9 * d)), DevBuf(ctx, 9 * d * 4)
    other_cache = blk.new_cache()

    def step():
        _ffi.check(_ffi.lib.pg_kv_cache_rollback_to(cache._h, pre))
        _ffi.check(_ffi.lib.pg_llama_block_forward_dev(ctx.handle, blk._h, h_dev.ptr, seq, cache._h, o_dev.ptr))

    def eager(x):
        _ffi.check(_ffi.lib.pg_memcpy_h2d(ctx.handle, h_dev.ptr, C.c_void_p(x.ctypes.data), x.nbytes))
        step()
        ctx.sync()
        return o_dev.to_host(np.float32)

    want = [eager(x) for x in inputs]        # (also the warm-up: every buffer the step needs exists now)
    say(f"capturing a {seq}-token step, type {typ}")
    graph, ex = hip.capture(ctx.stream, step)
    try:
        for i, x in enumerate(inputs):
            # other work of the library on the stream, and a synchronisation, between the replays
            _ffi.check(_ffi.lib.pg_kv_cache_rollback_to(other_cache._h, 0))
            _ffi.check(_ffi.lib.pg_llama_block_forward_dev(ctx.handle, blk._h, other_in.ptr, 9, other_cache._h, other_out.ptr))
            _ffi.check(_ffi.lib.pg_memcpy_h2d(ctx.handle, h_dev.ptr, C.c_void_p(x.ctypes.data), x.nbytes))
            _ffi.check(_ffi.lib.pg_memcpy_h2d(ctx.handle, o_dev.ptr, C.c_void_p(np.full(seq * d, np.nan, np.float32).ctypes.data), seq * d * 4))
            ctx.sync()
            hip.ok(hip.lib.hipGraphLaunch(ex, ctx.stream), "hipGraphLaunch")
            ctx.sync()
            got = o_dev.to_host(np.float32)
            assert (got.view(np.uint32) == want[i].view(np.uint32)).all(), f"replay {i} differs from the eager step"
    finally:
        hip.lib.hipGraphExecDestroy(ex)
        hip.lib.hipGraphDestroy(graph)
    for w in ws:
        w.free()


def test_few_row_products_replayed_from_a_graph(ctx, orc):
    """The few-row products (W8A8 over 8 rows, Q4_0 over 5 and over 2 rows: one launch each after the rows'
    quantisation / digits) captured together, after one eager call has made their buffers."""
    from peregrine_amd import _ffi, gguf, quant
    hip = Hip()
    k, n = 1024, 520
    qt = quant.quantize_weights(orc.rng_normal(31, k * n, 0.0, 0.02), k, n, ctx).to_gpu(ctx)
    gw = gguf.GgufWeight(bytes(H.pack_q4_0(orc.rng_normal(32, n * k, 0.0, 0.03))), 2, n, k, ctx)
    inputs = [orc.rng_normal(40 + i, 8 * k) for i in range(3)]
    x = DevBuf(ctx, host=inputs[0])
    outs = [DevBuf(ctx, 8 * n * 4) for _ in range(3)]

    def step():
        _ffi.check(_ffi.lib.pg_matmul_quantized_dev(ctx.handle, x.ptr, 8, k, qt._gpu, outs[0].ptr, None))
        _ffi.check(_ffi.lib.pg_gguf_matmul_dev(ctx.handle, x.ptr, 5, gw._h, outs[1].ptr))
        _ffi.check(_ffi.lib.pg_gguf_matmul_dev(ctx.handle, x.ptr, 2, gw._h, outs[2].ptr))

    def eager(v):
        _ffi.check(_ffi.lib.pg_memcpy_h2d(ctx.handle, x.ptr, C.c_void_p(v.ctypes.data), v.nbytes))
        step()
        ctx.sync()
        return [o.to_host(np.float32) for o in outs]

    want = [eager(v) for v in inputs]
    say("capturing three few-row products")
    graph, ex = hip.capture(ctx.stream, step)
    try:
        for i, v in enumerate(inputs):
            _ffi.check(_ffi.lib.pg_gguf_matmul_dev(ctx.handle, x.ptr, 1, gw._h, outs[1].ptr))   # other work in between
            _ffi.check(_ffi.lib.pg_memcpy_h2d(ctx.handle, x.ptr, C.c_void_p(v.ctypes.data), v.nbytes))
            for o in outs:
                _ffi.check(_ffi.lib.pg_memcpy_h2d(ctx.handle, o.ptr, C.c_void_p(np.full(8 * n, np.nan, np.float32).ctypes.data), 8 * n * 4))
            ctx.sync()
            hip.ok(hip.lib.hipGraphLaunch(ex, ctx.stream), "hipGraphLaunch")
            ctx.sync()
            for j, rows in enumerate((8, 5, 2)):
                got = outs[j].to_host(np.float32)[: rows * n]
                assert (got.view(np.uint32) == want[i][j][: rows * n].view(np.uint32)).all(), f"replay {i}, product {j} differs from the eager call"
    finally:
        hip.lib.hipGraphExecDestroy(ex)
        hip.lib.hipGraphDestroy(graph)
    gw.free()


def test_mxfp4_products_and_moe_replayed_from_a_graph(ctx, orc):
    """MXFP4 over many rows (digit records, tiles over two runs of K, their sum) and the gpt-oss MoE layer over
    MXFP4 experts in both its forms (token tiles of all experts in one launch; pair by pair for a few pairs),
    captured together after one eager call has made the buffers and the experts' pointer table."""
    from peregrine_amd import _ffi, mxfp4
    from test_oracle_formats_pins import _mx_expert
    hip = Hip()
    rng = np.random.default_rng(5)
    n, k, m = 600, 2048, 40
    w = mxfp4.upload(rng.integers(0, 256, n * k // 2, dtype=np.uint8), rng.integers(110, 130, n * k // 32, dtype=np.uint8), n, k, ctx)
    hidden, inter, E, top_k, T = 256, 128, 8, 2, 48
    experts = [mxfp4.Mxfp4Expert(hidden, inter, 1.702, 7.0, *_mx_expert(rng, hidden, inter), ctx=ctx) for _ in range(E)]
    tab = (C.c_void_p * E)(*[e._h.value for e in experts])
    idx = np.stack([rng.permutation(E)[:top_k] for _ in range(T)]).astype(np.int32)
    wt = rng.random((T, top_k)).astype(np.float32)
    inputs = [orc.rng_normal(60 + i, max(m * k, T * hidden)) for i in range(3)]
    x = DevBuf(ctx, host=inputs[0])
    d_idx, d_wt = DevBuf(ctx, host=idx), DevBuf(ctx, host=wt)
    outs = [DevBuf(ctx, m * n * 4), DevBuf(ctx, T * hidden * 4), DevBuf(ctx, 3 * hidden * 4)]
    sizes = [m * n, T * hidden, 3 * hidden]

    def step():
        _ffi.check(_ffi.lib.pg_gguf_matmul_dev(ctx.handle, x.ptr, m, w._h, outs[0].ptr))
        _ffi.check(_ffi.lib.pg_mxfp4_moe_ffn_routed_dev(ctx.handle, x.ptr, T, d_idx.ptr, d_wt.ptr, top_k, C.cast(tab, C.POINTER(C.c_void_p)), E, outs[1].ptr))
        _ffi.check(_ffi.lib.pg_mxfp4_moe_ffn_routed_dev(ctx.handle, x.ptr, 3, d_idx.ptr, d_wt.ptr, top_k, C.cast(tab, C.POINTER(C.c_void_p)), E, outs[2].ptr))

    def eager(v):
        _ffi.check(_ffi.lib.pg_memcpy_h2d(ctx.handle, x.ptr, C.c_void_p(v.ctypes.data), v.nbytes))
        ctx.profile_begin()
        step()
        prof = ctx.profile_end()
        ctx.sync()
        return [o.to_host(np.float32) for o in outs], prof

    want, prof = zip(*[eager(v) for v in inputs])
    assert {"mxfp4_tiles", "gguf_mm_sum_parts", "mxfp4_tiles_grouped", "mxfp4_rows_pairs"} <= set(prof[0]), prof[0]
    say("capturing an MXFP4 product and two MoE layers")
    graph, ex = hip.capture(ctx.stream, step)
    try:
        for i, v in enumerate(inputs):
            _ffi.check(_ffi.lib.pg_gguf_matmul_dev(ctx.handle, x.ptr, 1, w._h, outs[0].ptr))   # other work in between
            _ffi.check(_ffi.lib.pg_memcpy_h2d(ctx.handle, x.ptr, C.c_void_p(v.ctypes.data), v.nbytes))
            for o, sz in zip(outs, sizes):
                _ffi.check(_ffi.lib.pg_memcpy_h2d(ctx.handle, o.ptr, C.c_void_p(np.full(sz, np.nan, np.float32).ctypes.data), sz * 4))
            ctx.sync()
            hip.ok(hip.lib.hipGraphLaunch(ex, ctx.stream), "hipGraphLaunch")
            ctx.sync()
            for j in range(3):
                got = outs[j].to_host(np.float32)
                assert (got.view(np.uint32) == want[i][j].view(np.uint32)).all(), f"replay {i}, call {j} differs from the eager call"
    finally:
        hip.lib.hipGraphExecDestroy(ex)
        hip.lib.hipGraphDestroy(graph)
    w.free()
    for e in experts:
        e.free()
