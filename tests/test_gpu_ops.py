"""GPU parity of every kernel entry point against the CPU oracle on the same
seeded inputs, through the C-ABI.  Integer/byte work (conversion, gather,
argmax) is bit-exact; floating-point ops stay inside the 2e-2 max-abs/rel
tolerance the task states, and tighter bounds are asserted where the kernel
was built to reproduce the oracle's bits (RMSNorm, RoPE, residual)."""
import ctypes as C

import numpy as np
import pytest

from oracle import pyoracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
TOL = H.TOL
# projections: fp32 accumulation in a different order moves a result by at most one fp16 rounding step
# (9.8e-4 at magnitude 1..2, relative above), twice that with the residual's second rounding
TIGHT = 4e-3


def say(*a):
    print(*a, flush=True)


# ---- BF16 -> FP16: bit-exact -----------------------------------------------------------------
def test_convert_all_65536_patterns(gpu):
    src = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    assert np.array_equal(gpu.ops.bf16_to_fp16(src), orc.bf16_to_fp16(src))


@pytest.mark.parametrize("n", [0, 1, 7, 8, 9, 1000003])
def test_convert_ragged_sizes(gpu, n):
    rng = np.random.default_rng(n)
    src = rng.integers(0, 65536, size=n, dtype=np.uint32).astype(np.uint16)
    if n == 0:
        assert gpu.lib().llm_bf16_to_fp16(1, 1, 0, None) == 0
        return
    assert np.array_equal(gpu.ops.bf16_to_fp16(src), orc.bf16_to_fp16(src))


def test_convert_between_unaligned_buffers(gpu):
    """Source and destination that do not start on a 16-byte boundary take the element-wise kernel."""
    n = 100003
    src = np.random.default_rng(4).integers(0, 65536, size=n + 9, dtype=np.uint32).astype(np.uint16)
    d_src, d_dst = gpu.capi.DevBuf.from_host(src), gpu.capi.DevBuf.from_host(np.zeros(n + 9, np.uint16))
    gpu.capi.check(gpu.lib().llm_bf16_to_fp16(d_src.ptr + 2, d_dst.ptr + 6, n, None))
    out = d_dst.download()
    assert np.array_equal(out[3:3 + n], orc.bf16_to_fp16(src[1:1 + n]))
    assert not out[:3].any() and not out[3 + n:].any()


def test_convert_llama3_8b_ffn_tensor(gpu):
    # 4096 x 14336 seeded N(0, 0.02) bf16
    src = gpu.engine.seeded_normal_bf16(42, 7, 4096 * 14336)
    say("convert 4096x14336")
    assert np.array_equal(gpu.ops.bf16_to_fp16(src), orc.bf16_to_fp16(src))


# ---- embedding: exact ----------------------------------------------------------------------------
def test_embed_gather_exact_and_bad_id_is_nan(gpu):
    rng = np.random.default_rng(1)
    table = H.bits(rng.standard_normal((1000, 4096)))
    ids = np.array([5, 999, 0, 5, 123], np.int32)
    assert np.array_equal(gpu.ops.embed_gather(table, ids), orc.embed(table, ids))
    out = gpu.ops.embed_gather(table, np.array([1000, -1, 3], np.int32))
    assert np.all(out[:2] == 0x7fff) and np.array_equal(out[2], table[3])


# ---- RMSNorm ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,d", [(1, 4096), (128, 4096), (8192, 4096), (3, 256), (2, 512), (2, 16384)])
def test_rmsnorm(gpu, T, d):
    rng = np.random.default_rng(T + d)
    x = H.bits(rng.standard_normal((T, d)))
    g = H.bits(1.0 + 0.1 * rng.standard_normal(d))
    say("rmsnorm", T, d)
    got, want = gpu.ops.rmsnorm(x, g), orc.rmsnorm(x, g)
    mism = float(np.mean(got != want))
    say("  mismatching elements:", mism, "max ulp:", int(H.ulp_diff(got, want).max()))
    assert H.mixed_err(got, want) <= TOL
    assert np.array_equal(got, want)  # same summation tree, same eps promotion, correctly rounded divide
    assert np.array_equal(gpu.ops.rmsnorm(x, g, inplace=True), want)


def test_rmsnorm_rejects_unsupported_width(gpu):
    with pytest.raises(gpu.LlmError):
        gpu.ops.rmsnorm(np.zeros((1, 96), np.uint16), np.zeros(96, np.uint16))


def test_add_residual(gpu):
    rng = np.random.default_rng(3)
    for n in (8, 4096 * 5, 1001 * 8 + 3):
        a, b = H.bits(rng.standard_normal(n)), H.bits(rng.standard_normal(n))
        assert np.array_equal(gpu.ops.add_residual(a, b), orc.add(a, b))


# ---- RoPE ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T", [1, 128, 8192])
def test_rope_q_and_k_shapes(gpu, T):
    rng = np.random.default_rng(T)
    for heads in (32, 8):
        x = H.bits(rng.standard_normal((T, heads * 128)))
        say("rope", T, heads)
        got, want = gpu.ops.rope(x, heads, 128, 0), orc.rope(x, heads, 128, 0)
        say("  mismatching elements:", float(np.mean(got != want)))
        assert H.mixed_err(got, want) <= TOL
        assert np.array_equal(got, want)  # same libm table, unfused rotate


def test_rope_offset_and_small_head(gpu):
    rng = np.random.default_rng(5)
    x = H.bits(rng.standard_normal((9, 8 * 32)))
    assert np.array_equal(gpu.ops.rope(x, 8, 32, 50), orc.rope(x, 8, 32, 50))


@pytest.mark.parametrize("T,pos0", [(1, 0), (1, 77), (5, 3), (100, 28)])
def test_rope_kv_append_layouts(gpu, T, pos0):
    rng = np.random.default_rng(T * 100 + pos0)
    Hq, Hkv, hd, max_pos = 8, 2, 32, 128
    qd, kvd = Hq * hd, Hkv * hd
    qkv = H.bits(rng.standard_normal((T, qd + 2 * kvd)))
    q2, kc, vc = gpu.ops.rope_kv_append(qkv, Hq, Hkv, hd, pos0, max_pos)
    q_want = orc.rope(np.ascontiguousarray(qkv[:, :qd]), Hq, hd, pos0)
    k_want = orc.rope(np.ascontiguousarray(qkv[:, qd:qd + kvd]), Hkv, hd, pos0)
    assert np.array_equal(q2[:, :qd], q_want)
    assert np.array_equal(q2[:, qd:], qkv[:, qd:])  # K and V columns of the buffer are left alone
    kc_want = np.zeros_like(kc)
    vc_want = np.zeros_like(vc)
    kc_want[:, pos0:pos0 + T, :] = k_want.reshape(T, Hkv, hd).transpose(1, 0, 2)
    vc_want[:, :, pos0:pos0 + T] = qkv[:, qd + kvd:].reshape(T, Hkv, hd).transpose(1, 2, 0)
    assert np.array_equal(kc, kc_want) and np.array_equal(vc, vc_want)


# ---- projections at LLaMA3-8B layer shapes ----------------------------------------------------------------
SHAPES = {"qkv": (4096, 6144), "o": (4096, 4096), "down": (14336, 4096)}


def _proj_inputs(seed, T, K, N):
    rng = np.random.default_rng(seed)
    x = H.bits(rng.standard_normal((T, K)))
    w = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    return x, w


@pytest.mark.parametrize("name", list(SHAPES))
@pytest.mark.parametrize("T", [1, 4, 16])
def test_linear_skinny(gpu, name, T):
    K, N = SHAPES[name]
    x, w = _proj_inputs(T * 7 + K, T, K, N)
    say("linear", name, T)
    got, want = gpu.ops.linear(x, w), orc.linear(x, w)
    e = H.mixed_err(got, want)
    say("  err", e, "mismatch", float(np.mean(got != want)), "max ulp", int(H.ulp_diff(got, want).max()))
    assert e <= TIGHT


@pytest.mark.parametrize("tiles", [30, 100, 140, 256 + 40, 256 + 128, 256 + 200, 2 * 256 + 31])
@pytest.mark.parametrize("T", [2, 5, 16])
def test_skinny_tile_counts_around_the_cu_count(gpu, tiles, T):
    """The 2..16-row kernel walks persistently over 16-column tiles, one workgroup per CU: tile counts below, at
    and above multiples of the CU count (last rounds that are nearly empty, half full, nearly full) all write every
    output column once and match the oracle, with and without the residual and through the SwiGLU epilogue."""
    K, N = 1024, 16 * tiles
    rng = np.random.default_rng(tiles * 31 + T)
    x = H.bits(rng.standard_normal((T, K)))
    w = H.bits(0.05 * rng.standard_normal((N, K), dtype=np.float32))
    w2 = H.bits(0.05 * rng.standard_normal((N, K), dtype=np.float32))
    res = H.bits(rng.standard_normal((T, N)))
    say("skinny tiles", tiles, T)
    got = gpu.ops.linear(x, w, residual=res)
    assert H.mixed_err(got, orc.add(orc.linear(x, w), res)) <= TIGHT
    assert np.array_equal(gpu.ops.linear(x, w, residual=res, inplace=True), got)   # out == residual, as the engine calls it
    assert H.mixed_err(gpu.ops.linear(x, w), orc.linear(x, w)) <= TIGHT
    assert H.mixed_err(gpu.ops.linear_swiglu(x, w, w2), orc.linear_swiglu(x, w, w2)) <= TIGHT


@pytest.mark.parametrize("T", [1, 4, 16])
def test_linear_residual_epilogue(gpu, T):
    K, N = 4096, 4096
    x, w = _proj_inputs(T + 99, T, K, N)
    res = H.bits(np.random.default_rng(T).standard_normal((T, N)))
    got = gpu.ops.linear(x, w, residual=res)
    want = orc.add(orc.linear(x, w), res)
    assert H.mixed_err(got, want) <= TIGHT


@pytest.mark.parametrize("T", [1, 4, 16])
def test_swiglu_skinny(gpu, T):
    K, N = 4096, 14336
    rng = np.random.default_rng(T + 5)
    x = H.bits(rng.standard_normal((T, K)))
    wg = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    wu = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    say("swiglu", T)
    got, want = gpu.ops.linear_swiglu(x, wg, wu), orc.linear_swiglu(x, wg, wu)
    e = H.mixed_err(got, want)
    say("  err", e, "max ulp", int(H.ulp_diff(got, want).max()))
    assert e <= TOL


@pytest.mark.parametrize("T,K,N", [(17, 256, 384), (33, 768, 256), (64, 256, 768), (100, 4096, 512),
                                   (128, 4096, 6144), (200, 512, 1040), (129, 64, 272), (300, 128, 1008),
                                   (1000, 256, 4112), (1025, 64, 272), (1100, 192, 528), (2100, 4096, 400),
                                   # enough 256 x 256 tiles for the four-wave kernel, ragged edges, 2..6 k-steps
                                   (1100, 128, 10000), (1030, 64, 12304), (1300, 192, 9232)])
def test_linear_gemm_ragged_shapes(gpu, T, K, N):
    x, w = _proj_inputs(T + K + N, T, K, N)
    res = H.bits(np.random.default_rng(1).standard_normal((T, N)))
    say("gemm", T, K, N)
    got, want = gpu.ops.linear(x, w), orc.linear(x, w)
    assert got.shape == (T, N)
    e = H.mixed_err(got, want)
    say("  err", e, "max ulp", int(H.ulp_diff(got, want).max()))
    assert e <= TIGHT
    got_r = gpu.ops.linear(x, w, residual=res)
    assert H.mixed_err(got_r, orc.add(orc.linear(x, w), res)) <= TOL


@pytest.mark.parametrize("what,T,K,N,ldo", [
    # output rows that are not a multiple of 8 bytes apart: the register-staged MFMA kernels (64x64 and 128x128 /
    # 128x64 tiles) instead of the direct-to-LDS ones
    ("linear", 100, 256, 272, 274), ("linear", 40, 256, 272, 274), ("swiglu", 100, 256, 272, 274),
    ("swiglu", 20, 256, 48, None),
    # 2..16 rows with K not a multiple of 1024: the skinny kernel that reads the weights through registers
    ("linear", 8, 768, 512, None), ("swiglu", 8, 768, 512, None),
    # gate/up with few output tiles and a long K at 64 and 128 rows: split k with the two-matrix reduction
    ("swiglu", 64, 4096, 256, None), ("swiglu", 128, 4096, 256, None),
    # the 256 x 256-tile kernel with output rows 8 but not 16 bytes apart: its 8-byte store epilogue (rows
    # 16 bytes apart take 16-byte stores)
    ("linear", 1100, 128, 10000, 10004), ("swiglu", 1030, 128, 5008, 5012)])
def test_kernel_families_off_the_main_paths(gpu, what, T, K, N, ldo):
    """Shapes chosen so that every kernel family of the projections is launched by some test (the 8B shapes
    only reach the direct-to-LDS and skinny-DMA kernels)."""
    rng = np.random.default_rng(T + K + N)
    x = H.bits(rng.standard_normal((T, K)))
    w = H.bits(0.05 * rng.standard_normal((N, K), dtype=np.float32))
    if what == "linear":
        got, want = gpu.ops.linear(x, w, ldo=ldo), orc.linear(x, w)
    else:
        w2 = H.bits(0.05 * rng.standard_normal((N, K), dtype=np.float32))
        got, want = gpu.ops.linear_swiglu(x, w, w2, ldo=ldo), orc.linear_swiglu(x, w, w2)
    assert got.shape == (T, N)
    assert H.mixed_err(got, want) <= TOL


def test_split_k_linear_on_two_streams_at_once(gpu):
    """Split-K projections (64 rows, few output tiles) issued on two streams without waiting in between:
    each stream has its own partial-sum buffer, so both results equal the single-stream result bit for bit."""
    L, cap = gpu.lib(), gpu.capi
    T, K, N = 64, 4096, 4096
    streams = []
    for _ in range(2):
        s = C.c_void_p()
        cap.check(L.llm_stream_create(C.byref(s)))
        streams.append(s)
    bufs, want = [], []
    for i in range(2):
        x, w = _proj_inputs(50 + i, T, K, N)
        want.append(gpu.ops.linear(x, w))   # default stream, alone
        bufs.append((cap.DevBuf.from_host(x), cap.DevBuf.from_host(w), cap.DevBuf((T, N), np.uint16)))
    for rep in range(20):
        for i in range(2):
            d_x, d_w, d_o = bufs[i]
            cap.check(L.llm_linear(d_x.ptr, K, d_w.ptr, None, 0, d_o.ptr, N, T, N, K, streams[i]))
    for s in streams:
        cap.check(L.llm_stream_sync(s))
    for i in range(2):
        assert np.array_equal(bufs[i][2].download(), want[i]), i
        assert H.mixed_err(want[i], orc.linear(*_proj_inputs(50 + i, T, K, N))) <= TIGHT
    for s in streams:
        cap.check(L.llm_stream_destroy(s))


def test_linear_gemm_reference_test_operand_pattern(gpu):
    # the operand pattern of the reference's tests/gemm.cu scaled to a shape the kernels take:
    # x[i][j] = (i*K + j) % 5 - 2, w likewise; exact in fp32, so any layout slip shows
    T, K, N = 40, 128, 64
    x = ((np.arange(T * K).reshape(T, K) % 5) - 2).astype(np.float64)
    w = ((np.arange(N * K).reshape(N, K) % 7) - 3).astype(np.float64)
    got = gpu.ops.linear(H.bits(x), H.bits(w))
    assert np.array_equal(got, H.bits(x @ w.T))
    assert np.array_equal(gpu.ops.linear(H.bits(x[:1]), H.bits(w)), H.bits(x[:1] @ w.T))
    assert np.array_equal(gpu.ops.linear(H.bits(x[:5]), H.bits(w)), H.bits(x[:5] @ w.T))


@pytest.mark.parametrize("T,K,N", [(130, 64, 80), (300, 512, 1008), (1030, 128, 336), (1500, 4096, 208),
                                   (1030, 128, 5008), (1500, 64, 4112)])
def test_swiglu_gemm_ragged_shapes(gpu, T, K, N):
    rng = np.random.default_rng(T + N)
    x = H.bits(rng.standard_normal((T, K)))
    wg = H.bits(0.05 * rng.standard_normal((N, K), dtype=np.float32))
    wu = H.bits(0.05 * rng.standard_normal((N, K), dtype=np.float32))
    say("swiglu gemm", T, K, N)
    got, want = gpu.ops.linear_swiglu(x, wg, wu), orc.linear_swiglu(x, wg, wu)
    assert got.shape == (T, N)
    assert H.mixed_err(got, want) <= TIGHT


@pytest.mark.parametrize("name", list(SHAPES))
def test_linear_mfma_512(gpu, name):
    K, N = SHAPES[name]
    x, w = _proj_inputs(512 + K, 512, K, N)
    say("mfma 512", name)
    got, want = gpu.ops.linear(x, w), orc.linear(x, w)
    e = H.mixed_err(got, want)
    say("  err", e, "max ulp", int(H.ulp_diff(got, want).max()))
    assert e <= TIGHT


def test_swiglu_mfma_512(gpu):
    K, N, T = 4096, 14336, 512
    rng = np.random.default_rng(8)
    x = H.bits(rng.standard_normal((T, K)))
    wg = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    wu = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    got, want = gpu.ops.linear_swiglu(x, wg, wu), orc.linear_swiglu(x, wg, wu)
    e = H.mixed_err(got, want)
    say("swiglu 512 err", e)
    assert e <= TOL


def test_linear_mfma_8192_rows_sampled(gpu):
    # full T = 8192 on the GPU; the oracle follows 96 of the rows (rows are independent)
    K, N, T = 4096, 6144, 8192
    x, w = _proj_inputs(77, T, K, N)
    got = gpu.ops.linear(x, w)
    rows = np.r_[0:32, 4080:4112, 8160:8192]
    want = orc.linear(np.ascontiguousarray(x[rows]), w)
    e = H.mixed_err(got[rows], want)
    say("mfma 8192 err", e)
    assert e <= TIGHT
    # linearity in x at full size: doubling x doubles every fp32 sum exactly
    # (outputs that round into the fp16 subnormal range lose the doubled bit: left out)
    x2 = H.bits(2.0 * H.f16(x))
    a, b = H.f16(gpu.ops.linear(x2, w)), 2.0 * H.f16(got)
    normal = np.abs(b) >= 2.0 ** -12
    assert np.array_equal(a[normal], b[normal])


SAMPLED_ROWS = np.r_[0:32, 4080:4112, 8160:8192]   # first, middle and last row tiles of an 8192-row pass


def test_o_projection_mfma_8192_rows_sampled(gpu):
    """O projection of the 8192-token pass (K 4096 -> N 4096) with the residual added in place, as the engine
    calls it; the oracle follows 96 of the rows."""
    K, N, T = 4096, 4096, 8192
    x, w = _proj_inputs(78, T, K, N)
    res = H.bits(np.random.default_rng(79).standard_normal((T, N)))
    got = gpu.ops.linear(x, w, residual=res, inplace=True)
    want = orc.add(orc.linear(np.ascontiguousarray(x[SAMPLED_ROWS]), w), np.ascontiguousarray(res[SAMPLED_ROWS]))
    e = H.mixed_err(got[SAMPLED_ROWS], want)
    say("O 8192 err", e)
    assert e <= TIGHT
    assert np.array_equal(got, gpu.ops.linear(x, w, residual=res))   # in place == separate residual buffer


def test_down_projection_mfma_8192_rows_sampled(gpu):
    """Down projection of the 8192-token pass (K 14336 -> N 4096), residual in place."""
    K, N, T = 14336, 4096, 8192
    rng = np.random.default_rng(80)
    x = H.bits(rng.standard_normal((T, K), dtype=np.float32))
    w = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    res = H.bits(rng.standard_normal((T, N), dtype=np.float32))
    got = gpu.ops.linear(x, w, residual=res, inplace=True)
    want = orc.add(orc.linear(np.ascontiguousarray(x[SAMPLED_ROWS]), w), np.ascontiguousarray(res[SAMPLED_ROWS]))
    e = H.mixed_err(got[SAMPLED_ROWS], want)
    say("down 8192 err", e)
    assert e <= TIGHT


def test_swiglu_mfma_8192_rows_sampled(gpu):
    """Gate/up + SwiGLU of the 8192-token pass (K 4096 -> N 2 x 14336)."""
    K, N, T = 4096, 14336, 8192
    rng = np.random.default_rng(81)
    x = H.bits(rng.standard_normal((T, K), dtype=np.float32))
    wg = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    wu = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    got = gpu.ops.linear_swiglu(x, wg, wu)
    want = orc.linear_swiglu(np.ascontiguousarray(x[SAMPLED_ROWS]), wg, wu)
    e = H.mixed_err(got[SAMPLED_ROWS], want)
    say("swiglu 8192 err", e)
    assert e <= TOL


# ---- LM head + argmax -----------------------------------------------------------------------------------------
def test_lmhead_argmax_full_vocab(gpu):
    K, V = 4096, 128256
    rng = np.random.default_rng(9)
    x = H.bits(rng.standard_normal((1, K)))
    w = H.bits(0.02 * rng.standard_normal((V, K), dtype=np.float32))
    say("lm head")
    tok, logits = gpu.ops.lmhead_argmax(x, w)
    want = orc.linear(x, w).reshape(-1)
    e = H.mixed_err(logits, want)
    say("  err", e, "token", tok, orc.argmax_f16(want))
    assert e <= TIGHT
    assert tok == orc.argmax_f16(logits)  # argmax over the kernel's own fp16 logits: exact


def test_argmax_ties_zero_signs_nan(gpu):
    b = H.bits
    cases = [b([1.0, 3.0, 3.0, 2.0]), b([-0.0, 0.0, -1.0]), b([0.0, -0.0]), b([-np.inf, -5.0]),
             np.array([0x7e00, 0xfe00], np.uint16), np.array([0x3c00, 0x7e00, 0x3800], np.uint16)]
    rng = np.random.default_rng(10)
    big = b(rng.standard_normal(128256))
    big[[77, 90000]] = big.view(np.float16).max().view(np.uint16)  # a tie far apart: lowest index wins
    cases.append(big)
    cases.append(b(np.round(rng.standard_normal(300000) * 4) / 4))  # many ties
    for c in cases:
        assert gpu.ops.argmax_f16(c) == orc.argmax_f16(c)


@pytest.mark.parametrize("rows,n", [(1, 5), (4, 4096), (16, 128256), (3, 300001)])
def test_argmax_rows_matches_row_by_row(gpu, rows, n):
    rng = np.random.default_rng(rows * 1000 + n)
    m = H.bits(np.round(rng.standard_normal((rows, n)) * 8) / 8)  # many ties: the lowest index must win in every row
    got = gpu.ops.argmax_f16_rows(m)
    assert list(got) == [orc.argmax_f16(m[r]) for r in range(rows)]


# ---- attention ----------------------------------------------------------------------------------------------------
def _attn_inputs(seed, P, Hq, Hkv, hd):
    rng = np.random.default_rng(seed)
    return (H.bits(rng.standard_normal((P, Hq * hd))), H.bits(rng.standard_normal((P, Hkv * hd))),
            H.bits(rng.standard_normal((P, Hkv * hd))))


@pytest.mark.parametrize("ctx,max_pos", [(1, 64), (2, 64), (63, 64), (64, 64), (65, 2048), (384, 2048),
                                         (2048, 2048), (8448, 8704), (8704, 8704)])
def test_attn_decode_llama3_8b_heads(gpu, ctx, max_pos):
    Hq, Hkv, hd = 32, 8, 128
    q, k, v = _attn_inputs(ctx, ctx, Hq, Hkv, hd)
    kc, vc = gpu.ops.kv_layout(k, v, Hkv, hd, max_pos)
    # rows past ctx hold stale junk from an earlier, longer sequence
    kc[:, ctx:, :] = H.bits(np.float16(3.0))
    vc[:, :, ctx:] = H.bits(np.float16(-7.0))
    say("attn decode", ctx, max_pos)
    got = gpu.ops.attn_decode(q[-1], kc, vc, ctx, Hq, Hkv, hd, repeats=2)
    want = orc.attention(q[-1:], k, v, ctx - 1, Hq, Hkv, hd).reshape(-1)
    e = H.mixed_err(got, want)
    say("  err", e, "max ulp", int(H.ulp_diff(got, want).max()))
    assert e <= TOL


@pytest.mark.parametrize("ctx,Hq,Hkv,hd", [(300, 16, 2, 128), (700, 16, 2, 128), (400, 4, 4, 128), (1500, 4, 4, 128),
                                          (260, 8, 2, 64), (900, 8, 2, 64), (513, 2, 2, 32), (40, 4, 4, 64)])
def test_attn_decode_other_head_shapes(gpu, ctx, Hq, Hkv, hd):
    """llm_attn_decode (queries already rotated, token already in the cache) for the group sizes and head sizes
    besides the 8B one: one span, two blocks per wavefront, several spans merged by the last workgroup."""
    q, k, v = _attn_inputs(ctx + Hq, ctx, Hq, Hkv, hd)
    kc, vc = gpu.ops.kv_layout(k, v, Hkv, hd, 2048)
    say("attn decode", ctx, Hq, Hkv, hd)
    got = gpu.ops.attn_decode(q[-1], kc, vc, ctx, Hq, Hkv, hd, repeats=2)
    want = orc.attention(q[-1:], k, v, ctx - 1, Hq, Hkv, hd).reshape(-1)
    e = H.mixed_err(got, want)
    say("  err", e)
    assert e <= TOL


def test_attn_decode_small_heads_and_gqa_map(gpu):
    Hq, Hkv, hd, ctx = 8, 2, 32, 20
    q, k, v = _attn_inputs(3, ctx, Hq, Hkv, hd)
    # V rows constant per KV head: the output reveals which KV head each query head read
    v = H.bits(np.repeat(np.arange(1, Hkv + 1, dtype=np.float64)[None, :], ctx, 0).repeat(hd, 1))
    kc, vc = gpu.ops.kv_layout(k, v, Hkv, hd, 64)
    got = H.f16(gpu.ops.attn_decode(q[-1], kc, vc, ctx, Hq, Hkv, hd)).reshape(Hq, hd)
    for h in range(Hq):
        assert np.allclose(got[h], h // 4 + 1, atol=2e-3)


@pytest.mark.parametrize("T,pos0,max_pos,Hkv", [(64, 0, 128, 2), (200, 0, 256, 8), (130, 70, 256, 1), (1000, 24, 1024, 2)])
def test_attn_prefill_that_rotates_its_queries_equals_rope_then_attention(gpu, T, pos0, max_pos, Hkv):
    """llm_rope_k_append + llm_attn_prefill_rope_q (K rotated into the cache, V stored, the queries rotated inside
    the attention kernel as it loads them) against llm_rope_kv_append + llm_attn_prefill: same attention output and
    same caches bit for bit, the queries in the projection buffer left as they were, ragged last blocks and a
    prompt appended behind cached positions included; the oracle bounds the result."""
    hd, Hq = 128, 4 * Hkv
    rng = np.random.default_rng(T + pos0)
    qkv = H.bits(rng.standard_normal((T, (Hq + 2 * Hkv) * hd)))
    kc0 = np.zeros((Hkv, max_pos, hd), np.uint16)
    vc0 = np.zeros((Hkv, hd, max_pos), np.uint16)
    if pos0:
        kc0[:, :pos0] = H.bits(rng.standard_normal((Hkv, pos0, hd)))
        vc0[:, :, :pos0] = H.bits(rng.standard_normal((Hkv, hd, pos0)))
    say("attn prefill with its own rope", T, pos0, max_pos, Hkv)
    assert gpu.lib().llm_attn_prefill_rope_q_supported(T, Hq, Hkv, hd, max_pos) == 1
    q_rot, kc_r, vc_r = gpu.ops.rope_kv_append(qkv, Hq, Hkv, hd, pos0, max_pos, kc=kc0, vc=vc0)
    want = gpu.ops.attn_prefill(q_rot[:, :Hq * hd].copy(), kc_r, vc_r, pos0, Hq, Hkv, hd)
    got, qkv_after, kc_f, vc_f = gpu.ops.rope_k_append_attn_prefill(qkv, Hq, Hkv, hd, pos0, max_pos, kc=kc0, vc=vc0)
    assert np.array_equal(kc_f, kc_r) and np.array_equal(vc_f, vc_r)
    assert np.array_equal(qkv_after, qkv)
    assert np.array_equal(got, want)
    assert gpu.lib().llm_attn_prefill_rope_q_supported(63, Hq, Hkv, hd, max_pos) == 0
    assert gpu.lib().llm_attn_prefill_rope_q_supported(T, 8 * Hkv, Hkv, hd, max_pos) == 0


@pytest.mark.parametrize("T,pos0,Hq,Hkv,hd", [(1, 0, 8, 2, 32), (16, 0, 8, 2, 32), (33, 7, 8, 2, 32),
                                              (64, 0, 32, 8, 128), (100, 60, 32, 8, 128), (512, 0, 32, 8, 128),
                                              # fewer than 64 rows at the 8B head shape: the kernel of the short blocks
                                              (40, 9, 32, 8, 128),
                                              # several pipelined tiles before the masked ones, rows not a multiple of the
                                              # block, prompt continued at an unaligned position; other group sizes and head dims
                                              (300, 37, 32, 8, 128), (257, 129, 8, 2, 64), (200, 300, 8, 1, 128),
                                              (130, 5, 4, 4, 128), (321, 64, 16, 4, 32)])
def test_attn_prefill(gpu, T, pos0, Hq, Hkv, hd):
    P = pos0 + T
    q, k, v = _attn_inputs(T + pos0, P, Hq, Hkv, hd)
    max_pos = (P + 63) // 64 * 64
    kc, vc = gpu.ops.kv_layout(k, v, Hkv, hd, max_pos)
    say("attn prefill", T, pos0, Hq, hd)
    got = gpu.ops.attn_prefill(q[pos0:], kc, vc, pos0, Hq, Hkv, hd)
    want = orc.attention(np.ascontiguousarray(q[pos0:]), k, v, pos0, Hq, Hkv, hd)
    e = H.mixed_err(got, want)
    say("  err", e, "max ulp", int(H.ulp_diff(got, want).max()))
    assert e <= TOL


@pytest.mark.parametrize("T,pos0,shape", [(448, 0, "rising"), (448, 0, "falling"), (300, 37, "spikes"),
                                          (448, 64, "flat")])
def test_attn_prefill_score_ranges_that_move_the_softmax_reference(gpu, T, pos0, shape):
    """The pipelined kernel (head size 128, group 4, 64 rows and more) keeps one softmax reference per query and
    moves it only when a probability would overflow fp16.  Key magnitudes that rise along the sequence force that
    move again and again; falling ones leave every later probability far below the reference; spikes put single
    scores 2^30 above their neighbours; all-equal keys keep every probability at exactly 1."""
    Hq, Hkv, hd = 32, 8, 128
    P = pos0 + T
    rng = np.random.default_rng(T + pos0)
    q = rng.standard_normal((P, Hq * hd))
    k = rng.standard_normal((P, Hkv * hd))
    v = rng.standard_normal((P, Hkv * hd))
    ramp = np.linspace(0.05, 6.0, P)[:, None]
    if shape == "rising":
        k *= ramp
    elif shape == "falling":
        k *= ramp[::-1]
    elif shape == "spikes":
        k[rng.integers(0, P, size=12)] *= 9.0
    else:
        k[:] = k[:1]
    q, k, v = H.bits(q), H.bits(k), H.bits(v)
    max_pos = (P + 63) // 64 * 64
    kc, vc = gpu.ops.kv_layout(k, v, Hkv, hd, max_pos)
    say("attn prefill", shape, T, pos0)
    got = gpu.ops.attn_prefill(q[pos0:], kc, vc, pos0, Hq, Hkv, hd)
    want = orc.attention(np.ascontiguousarray(q[pos0:]), k, v, pos0, Hq, Hkv, hd)
    e = H.mixed_err(got, want)
    say("  err", e, "max ulp", int(H.ulp_diff(got, want).max()))
    assert e <= TOL


def test_attn_prefill_8192_last_rows_and_uniform_key_property(gpu):
    T, Hq, Hkv, hd = 8192, 32, 8, 128
    q, k, v = _attn_inputs(11, T, Hq, Hkv, hd)
    kc, vc = gpu.ops.kv_layout(k, v, Hkv, hd, T)
    say("attn prefill 8192")
    got = gpu.ops.attn_prefill(q, kc, vc, 0, Hq, Hkv, hd)
    # oracle on the first rows and on a late chunk
    want0 = orc.attention(np.ascontiguousarray(q[:64]), k, v, 0, Hq, Hkv, hd)
    assert H.mixed_err(got[:64], want0) <= TOL
    want1 = orc.attention(np.ascontiguousarray(q[8128:8160]), k, v, 8128, Hq, Hkv, hd)
    e = H.mixed_err(got[8128:8160], want1)
    say("  late rows err", e)
    assert e <= TOL
    # size-independent property: identical keys => row i is the mean of V[0..i]
    k1 = np.tile(k[:1], (T, 1))
    kc1, _ = gpu.ops.kv_layout(k1, v, Hkv, hd, T)
    out = H.f16(gpu.ops.attn_prefill(q, kc1, vc, 0, Hq, Hkv, hd))
    vf = H.f16(v)
    csum = np.cumsum(vf, axis=0) / np.arange(1, T + 1)[:, None]
    for h in (0, 5, 31):
        kv = h // 4
        assert np.allclose(out[:, h * hd:(h + 1) * hd], csum[:, kv * hd:(kv + 1) * hd], atol=5e-3)


# ---- the decode step's fused entry points give the bits of the unfused sequence ------------------------------
@pytest.mark.parametrize("K,N", [(4096, 6144), (256, 384)])
def test_norm_linear_equals_rmsnorm_then_linear(gpu, K, N):
    rng = np.random.default_rng(K)
    x = H.bits(2.0 * rng.standard_normal((1, K)))
    g = H.bits(1.0 + 0.1 * rng.standard_normal(K))
    w = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    got = gpu.ops.norm_linear(x, g, w)
    assert np.array_equal(got, gpu.ops.linear(gpu.ops.rmsnorm(x, g), w))
    assert H.mixed_err(got, orc.linear(orc.rmsnorm(x, g), w)) <= TIGHT


@pytest.mark.parametrize("K,N,vocab", [(4096, 6144, 1000), (256, 384, 50), (4096, 100, 7)])
def test_embed_norm_linear_equals_gather_then_norm_linear(gpu, K, N, vocab):
    """The first projection of a decode step with the gather folded in: the row it leaves is the table's row, the
    projection has the bits of llm_embed_gather + llm_norm_linear, the id is read at ids[*offset], and an id
    outside the table gives the gather's NaN row and a NaN projection."""
    rng = np.random.default_rng(K + N)
    table = H.bits(2.0 * rng.standard_normal((vocab, K)))
    g = H.bits(1.0 + 0.1 * rng.standard_normal(K))
    w = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    ids = np.array([3, vocab - 1, 0, vocab, -1, 5], np.int32)
    for off in (None, 0, 1, 2, 5):
        say("embed_norm_linear", K, N, vocab, "offset", off)
        tok = int(ids[off or 0])
        got, row = gpu.ops.embed_norm_linear(table, ids, off, g, w)
        assert np.array_equal(row, table[tok])
        x = gpu.ops.embed_gather(table, np.array([tok], np.int32))
        assert np.array_equal(got, gpu.ops.norm_linear(x, g, w))
        assert H.mixed_err(got, orc.linear(orc.rmsnorm(orc.embed(table, [tok]), g), w)) <= TIGHT
    for off in (3, 4):
        say("embed_norm_linear", K, N, vocab, "bad id at offset", off)
        got, row = gpu.ops.embed_norm_linear(table, ids, off, g, w)
        assert np.all(row == 0x7fff)
        x = gpu.ops.embed_gather(table, ids[off:off + 1])
        assert np.array_equal(got, gpu.ops.norm_linear(x, g, w)) and np.all(np.isnan(H.f16(got)))


@pytest.mark.parametrize("K,N", [(4096, 14336), (256, 768)])
def test_norm_linear_swiglu_equals_unfused(gpu, K, N):
    rng = np.random.default_rng(K + 1)
    x = H.bits(2.0 * rng.standard_normal((1, K)))
    g = H.bits(1.0 + 0.1 * rng.standard_normal(K))
    wg = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    wu = H.bits(0.02 * rng.standard_normal((N, K), dtype=np.float32))
    got = gpu.ops.norm_linear_swiglu(x, g, wg, wu)
    assert np.array_equal(got, gpu.ops.linear_swiglu(gpu.ops.rmsnorm(x, g), wg, wu))
    assert H.mixed_err(got, orc.linear_swiglu(orc.rmsnorm(x, g), wg, wu)) <= TOL


def test_norm_lmhead_argmax_equals_unfused(gpu):
    K, V = 4096, 128256
    rng = np.random.default_rng(13)
    x = H.bits(3.0 * rng.standard_normal((1, K)))
    g = H.bits(1.0 + 0.1 * rng.standard_normal(K))
    w = H.bits(0.02 * rng.standard_normal((V, K), dtype=np.float32))
    tok, logits = gpu.ops.norm_lmhead_argmax(x, g, w)
    tok2, logits2 = gpu.ops.lmhead_argmax(gpu.ops.rmsnorm(x, g), w)
    assert tok == tok2 == orc.argmax_f16(logits) and np.array_equal(logits, logits2)


@pytest.mark.parametrize("pos,max_pos,Hq,Hkv,hd", [(0, 64, 8, 2, 32), (37, 64, 8, 2, 32), (0, 2048, 32, 8, 128),
                                                   (300, 2048, 32, 8, 128), (511, 2048, 32, 8, 128),
                                                   (512, 2048, 32, 8, 128), (1500, 2048, 32, 8, 128),
                                                   (8447, 8704, 32, 8, 128),
                                                   # long form around the points where its span length changes on a
                                                   # 256-CU device (spans of 256 up to 8192 positions, then growing
                                                   # in steps of 32 up to 512; beyond 16384 more than 32 spans)
                                                   (8191, 16640, 32, 8, 128), (8192, 16640, 32, 8, 128),
                                                   (12287, 16640, 32, 8, 128), (16383, 16640, 32, 8, 128),
                                                   (16600, 16640, 32, 8, 128),
                                                   # the other head shapes the kernels are built for: groups of 8 and
                                                   # of 1 at head size 128, head sizes 64 and 32, one and two blocks
                                                   # per wavefront, short and long form
                                                   (100, 1024, 16, 2, 128), (400, 1024, 16, 2, 128), (900, 1024, 16, 2, 128),
                                                   (300, 1024, 4, 4, 128), (700, 1024, 4, 4, 128),
                                                   (450, 1024, 8, 2, 64), (600, 1024, 8, 2, 64), (77, 1024, 4, 4, 64),
                                                   (500, 1024, 2, 2, 32), (1000, 1024, 2, 2, 32)])
def test_attn_decode_rope_fused(gpu, pos, max_pos, Hq, Hkv, hd):
    """RoPE + cache append + attention in one launch == llm_rope_kv_append then llm_attn_decode, and == oracle."""
    rng = np.random.default_rng(pos + hd)
    qd, kvd = Hq * hd, Hkv * hd
    # cache rows 0..pos-1 hold earlier (already rotated) keys and values
    k_old = H.bits(rng.standard_normal((pos, kvd)))
    v_old = H.bits(rng.standard_normal((pos, kvd)))
    kc, vc = gpu.ops.kv_layout(k_old, v_old, Hkv, hd, max_pos)
    qkv = H.bits(rng.standard_normal((1, qd + 2 * kvd)))
    say("attn decode fused", pos, max_pos)
    out, kc2, vc2 = gpu.ops.attn_decode_rope(qkv, kc, vc, pos, Hq, Hkv, hd, repeats=2)
    q_rot, kc_ref, vc_ref = gpu.ops.rope_kv_append(qkv, Hq, Hkv, hd, pos, max_pos, kc=kc, vc=vc)
    assert np.array_equal(kc2, kc_ref) and np.array_equal(vc2, vc_ref)
    ref = gpu.ops.attn_decode(q_rot[0, :qd], kc_ref, vc_ref, pos + 1, Hq, Hkv, hd)
    assert np.array_equal(out, ref)
    q_o = orc.rope(np.ascontiguousarray(qkv[:, :qd]), Hq, hd, pos)
    k_new = orc.rope(np.ascontiguousarray(qkv[:, qd:qd + kvd]), Hkv, hd, pos)
    k_all = np.concatenate([k_old, k_new], 0)
    v_all = np.concatenate([v_old, qkv[:, qd + kvd:]], 0)
    want = orc.attention(q_o, k_all, v_all, pos, Hq, Hkv, hd).reshape(-1)
    e = H.mixed_err(out, want)
    say("  err", e)
    assert e <= TOL
    # the two-launch long-context form: same caches, same result to rounding, at every position
    out_l, kc3, vc3 = gpu.ops.attn_decode_rope(qkv, kc, vc, pos, Hq, Hkv, hd, repeats=2, long_form=True)
    assert np.array_equal(kc3, kc_ref) and np.array_equal(vc3, vc_ref)
    e = H.mixed_err(out_l, want)
    say("  long form err", e)
    assert e <= TOL and H.mixed_err(out_l, out) <= TIGHT


@pytest.mark.parametrize("pos,max_pos,Hq,Hkv,hd,N", [(0, 64, 32, 8, 128, 4096), (700, 1024, 32, 8, 128, 4096),
                                                     (8300, 8704, 32, 8, 128, 4096), (300, 512, 32, 8, 128, 1008),
                                                     (137, 320, 8, 2, 32, 256), (530, 576, 4, 4, 64, 272),
                                                     (900, 1024, 16, 2, 128, 2048), (600, 1024, 4, 4, 128, 512),
                                                     (700, 1024, 8, 2, 64, 512), (1000, 1024, 2, 2, 32, 64)])
def test_attn_decode_rope_long_oproj_equals_the_three_launches(gpu, pos, max_pos, Hq, Hkv, hd, N):
    """Span kernel, then merge + output projection in one launch (the merge workgroups hand their heads over to
    the projection workgroups, which fetched their weights meanwhile): attention output, projection output (with
    the in-place residual) and both caches equal llm_attn_decode_rope_long followed by llm_linear bit for bit, on
    three calls in a row through the buffer ring, with no wait that ran into its limit."""
    rng = np.random.default_rng(pos + N + 1)
    qd, kvd = Hq * hd, Hkv * hd
    qkv = H.bits(rng.standard_normal((1, qd + 2 * kvd)))
    k_old, v_old = H.bits(rng.standard_normal((pos, kvd))), H.bits(rng.standard_normal((pos, kvd)))
    kc, vc = gpu.ops.kv_layout(k_old, v_old, Hkv, hd, max_pos)
    w = H.bits(0.05 * rng.standard_normal((N, qd)))
    res = H.bits(rng.standard_normal((1, N)))
    say("span, merge+oproj", pos, max_pos, Hq, Hkv, hd, N)
    assert gpu.lib().llm_attn_long_oproj_supported(Hq, Hkv, hd, N) == 1
    a_f, o_f, kc_f, vc_f, timeouts = gpu.ops.attn_decode_rope_oproj(qkv, kc, vc, pos, Hq, Hkv, hd, w, residual=res, repeats=3,
                                                                    long_form=True)
    assert timeouts == 0
    a_r, kc_r, vc_r = gpu.ops.attn_decode_rope(qkv, kc, vc, pos, Hq, Hkv, hd, long_form=True)
    o_r = gpu.ops.linear(a_r.reshape(1, -1), w, residual=res).reshape(-1)
    assert np.array_equal(a_f, a_r) and np.array_equal(kc_f, kc_r) and np.array_equal(vc_f, vc_r)
    assert np.array_equal(o_f, o_r), int(H.ulp_diff(o_f, o_r).max())
    want = orc.add(orc.linear(a_r.reshape(1, -1), w), res).reshape(-1)
    assert H.mixed_err(o_f, want) <= TOL
    _, o_n, _, _, timeouts = gpu.ops.attn_decode_rope_oproj(qkv, kc, vc, pos, Hq, Hkv, hd, w, long_form=True)
    assert timeouts == 0 and np.array_equal(o_n, gpu.ops.linear(a_r.reshape(1, -1), w).reshape(-1))


@pytest.mark.parametrize("pos,max_pos,Hq,Hkv,hd,N", [(0, 64, 32, 8, 128, 4096), (200, 1024, 32, 8, 128, 4096),
                                                     (511, 8704, 32, 8, 128, 4096), (300, 512, 32, 8, 128, 1008),
                                                     (37, 64, 8, 2, 32, 256), (130, 256, 4, 4, 64, 272),
                                                     (333, 512, 16, 2, 128, 2048), (60, 512, 4, 4, 128, 512),
                                                     (290, 512, 8, 2, 64, 512), (400, 512, 2, 2, 32, 64)])
def test_attn_decode_rope_oproj_equals_the_two_launches(gpu, pos, max_pos, Hq, Hkv, hd, N):
    """Attention + output projection in one launch (the projection's workgroups fetch their weights while
    the attention runs, then wait for it): attention output, projection output (with the in-place residual)
    and both caches equal llm_attn_decode_rope followed by llm_linear bit for bit, on three launches in a
    row through the counter ring, with no wait that ran into its limit; the oracle bounds the result."""
    rng = np.random.default_rng(pos + N)
    qd, kvd = Hq * hd, Hkv * hd
    qkv = H.bits(rng.standard_normal((1, qd + 2 * kvd)))
    k_old, v_old = H.bits(rng.standard_normal((pos, kvd))), H.bits(rng.standard_normal((pos, kvd)))
    kc, vc = gpu.ops.kv_layout(k_old, v_old, Hkv, hd, max_pos)
    w = H.bits(0.05 * rng.standard_normal((N, qd)))
    res = H.bits(rng.standard_normal((1, N)))
    say("attn+oproj", pos, max_pos, Hq, Hkv, hd, N)
    a_f, o_f, kc_f, vc_f, timeouts = gpu.ops.attn_decode_rope_oproj(qkv, kc, vc, pos, Hq, Hkv, hd, w, residual=res, repeats=3)
    assert timeouts == 0
    a_r, kc_r, vc_r = gpu.ops.attn_decode_rope(qkv, kc, vc, pos, Hq, Hkv, hd)
    o_r = gpu.ops.linear(a_r.reshape(1, -1), w, residual=res).reshape(-1)
    assert np.array_equal(a_f, a_r) and np.array_equal(kc_f, kc_r) and np.array_equal(vc_f, vc_r)
    assert np.array_equal(o_f, o_r), int(H.ulp_diff(o_f, o_r).max())
    want = orc.add(orc.linear(a_r.reshape(1, -1), w), res).reshape(-1)
    assert H.mixed_err(o_f, want) <= TOL
    # without a residual
    _, o_n, _, _, timeouts = gpu.ops.attn_decode_rope_oproj(qkv, kc, vc, pos, Hq, Hkv, hd, w)
    assert timeouts == 0 and np.array_equal(o_n, gpu.ops.linear(a_r.reshape(1, -1), w).reshape(-1))
