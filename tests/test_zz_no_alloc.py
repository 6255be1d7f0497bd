"""llm_attn_decode_noalloc (the entry point that allocates nothing: its partial results and counters
live in an array built into the library) against llm_attn_decode with a caller-supplied workspace,
through the C-ABI.  Same kernels on the same inputs, so the outputs must be equal bit for bit; the
oracle bounds both.  Collected last on purpose: a failure here must not hide other tests."""
import ctypes as C

import numpy as np
import pytest

from oracle import pyoracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _case(gpu, seed, ctx, max_pos, Hq, Hkv, hd):
    rng = np.random.default_rng(seed)
    q = H.bits(rng.standard_normal((ctx, Hq * hd)))
    k = H.bits(rng.standard_normal((ctx, Hkv * hd)))
    v = H.bits(rng.standard_normal((ctx, Hkv * hd)))
    kc, vc = gpu.ops.kv_layout(k, v, Hkv, hd, max_pos)
    print("noalloc case: seed", seed, "ctx", ctx, "max_pos", max_pos, "heads", Hq, Hkv, "hd", hd, flush=True)
    got = gpu.ops.attn_decode_noalloc(q[-1], kc, vc, ctx, Hq, Hkv, hd)
    ref = gpu.ops.attn_decode(q[-1], kc, vc, ctx, Hq, Hkv, hd)
    want = orc.attention(q[-1:], k, v, ctx - 1, Hq, Hkv, hd).reshape(-1)
    assert np.array_equal(got, ref), int(H.ulp_diff(got, ref).max())
    assert H.mixed_err(got, want) <= 4e-3


def test_noalloc_matches_workspace_entry_point_on_consecutive_calls(gpu):
    # the LLaMA3-8B head shape over four 512-position spans: partial results and counters in use
    _case(gpu, 1, 2048, 2048, 32, 8, 128)
    # a smaller input right after: its counters fall where the first call left partial sums
    _case(gpu, 2, 700, 1024, 8, 2, 64)
    # one span (no partial results), then the large shape again, then the tiny model's heads
    _case(gpu, 3, 100, 1024, 8, 2, 64)
    _case(gpu, 4, 1500, 2048, 32, 8, 128)
    _case(gpu, 5, 600, 1024, 8, 2, 32)


def _free_bytes(gpu):
    f, t = C.c_size_t(0), C.c_size_t(0)
    gpu.capi.check(gpu.lib().llm_mem_info(C.byref(f), C.byref(t)))
    return f.value


def test_noalloc_takes_no_device_memory_and_replays_from_a_captured_graph(gpu):
    """Free device memory is the same before and after calls of both span forms; one call recorded into a
    graph (which forbids allocation) gives the eager result on every one of four replays, with eager calls of
    another shape in between that leave other contents in the shared scratch array."""
    L = gpu.lib()
    Hq, Hkv, hd, max_pos, ctx = 32, 8, 128, 2048, 1700
    rng = np.random.default_rng(6)
    q = H.bits(rng.standard_normal((1, Hq * hd)))
    k, v = H.bits(rng.standard_normal((ctx, Hkv * hd))), H.bits(rng.standard_normal((ctx, Hkv * hd)))
    kc, vc = gpu.ops.kv_layout(k, v, Hkv, hd, max_pos)
    d_q, d_k, d_v = gpu.capi.DevBuf.from_host(q), gpu.capi.DevBuf.from_host(kc), gpu.capi.DevBuf.from_host(vc)
    d_o, d_o2 = gpu.capi.DevBuf((Hq * hd,), np.uint16), gpu.capi.DevBuf((Hq * hd,), np.uint16)
    stream = C.c_void_p()
    gpu.capi.check(L.llm_stream_create(C.byref(stream)))
    call = lambda out, n, s: gpu.capi.check(L.llm_attn_decode_noalloc(d_q.ptr, d_k.ptr, d_v.ptr, out.ptr, n, None, Hq, Hkv, hd,
                                                                      max_pos, s))
    call(d_o, ctx, stream)       # first use on this device (address look-up, module load) before the measurement
    gpu.capi.check(L.llm_stream_sync(stream))
    before = _free_bytes(gpu)
    for n in (ctx, 300, 900, ctx):
        call(d_o, n, stream)
    gpu.capi.check(L.llm_stream_sync(stream))
    assert _free_bytes(gpu) == before
    eager = d_o.download()
    # recorded once, replayed four times
    graph = C.c_void_p()
    gpu.capi.check(L.llm_graph_capture_begin(stream))
    call(d_o2, ctx, stream)
    gpu.capi.check(L.llm_graph_capture_end(stream, C.byref(graph)))
    for rep in range(4):
        d_o2.zero()
        call(d_o, 300 + 200 * rep, stream)    # eager work between the replays, other contents in the scratch array
        gpu.capi.check(L.llm_graph_launch(graph, stream))
        gpu.capi.check(L.llm_stream_sync(stream))
        assert np.array_equal(d_o2.download(), eager), rep
    gpu.capi.check(L.llm_graph_destroy(graph))
    gpu.capi.check(L.llm_stream_destroy(stream))
    print("free device bytes before", before, "after the graph was destroyed", _free_bytes(gpu), flush=True)


def test_noalloc_rejects_invalid_calls_before_launching_anything(gpu):
    """Arguments that llm_attn_decode refuses are refused by the no-allocation entry point as well, with
    nothing enqueued (checked under stream capture, where a launch would become a node of the graph)."""
    L = gpu.lib()
    buf = gpu.capi.DevBuf((32 * 128,), np.uint16)
    for args in ((buf.ptr, buf.ptr, buf.ptr, buf.ptr, 1, None, 32, 8, 128, 100, None),    # max_pos not a multiple of 64
                 (buf.ptr, buf.ptr, buf.ptr, buf.ptr, 65, None, 32, 8, 128, 64, None),    # ctx beyond max_pos
                 (buf.ptr, buf.ptr, buf.ptr, buf.ptr, 1, None, 32, 5, 128, 64, None),     # heads do not divide
                 (None, buf.ptr, buf.ptr, buf.ptr, 1, None, 32, 8, 128, 64, None),        # null pointer
                 (buf.ptr, buf.ptr, buf.ptr, buf.ptr, 1, None, 32, 8, 96, 64, None)):     # head size that is not built
        assert L.llm_attn_decode_noalloc(*args) == gpu.capi.LLM_ERR_INVALID, args


def test_noalloc_rejects_shapes_beyond_its_scratch(gpu):
    L = gpu.lib()
    assert L.llm_attn_decode_noalloc_max_bytes() == 4 * 32 * 256 * 130 + 4 * 32
    buf = gpu.capi.DevBuf((64 * 128,), np.uint16)
    rc = L.llm_attn_decode_noalloc(buf.ptr, buf.ptr, buf.ptr, buf.ptr, 1, None, 64, 8, 128, 64, None)
    assert rc == gpu.capi.LLM_ERR_INVALID and b"scratch" in L.llm_last_error()
    rc = L.llm_attn_decode_noalloc(buf.ptr, buf.ptr, buf.ptr, buf.ptr, 1, None, 32, 8, 256, 64, None)
    assert rc == gpu.capi.LLM_ERR_INVALID and b"scratch" in L.llm_last_error()
