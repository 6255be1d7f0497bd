"""llm_attn_decode_noalloc (the entry point that allocates nothing: its partial results and counters
live in an array built into the library) against llm_attn_decode with a caller-supplied workspace,
through the C-ABI.  Same kernels on the same inputs, so the outputs must be equal bit for bit; the
oracle bounds both.  Collected last on purpose: a failure here must not hide other tests."""
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


def test_noalloc_rejects_shapes_beyond_its_scratch(gpu):
    L = gpu.lib()
    assert L.llm_attn_decode_noalloc_max_bytes() == 4 * 32 * 256 * 130 + 4 * 32
    buf = gpu.capi.DevBuf((64 * 128,), np.uint16)
    rc = L.llm_attn_decode_noalloc(buf.ptr, buf.ptr, buf.ptr, buf.ptr, 1, None, 64, 8, 128, 64, None)
    assert rc == gpu.capi.LLM_ERR_INVALID and b"scratch" in L.llm_last_error()
    rc = L.llm_attn_decode_noalloc(buf.ptr, buf.ptr, buf.ptr, buf.ptr, 1, None, 32, 8, 256, 64, None)
    assert rc == gpu.capi.LLM_ERR_INVALID and b"scratch" in L.llm_last_error()
