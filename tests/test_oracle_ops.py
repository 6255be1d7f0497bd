"""Pins the CPU oracle op by op without the reference running (it cannot: it is
CUDA and holds no golden vectors).  Every check is one a plausible mistake
fails: closed forms in float64, invariants, special cases, brute force, and
the operand pattern of the reference's own tests/gemm.cu."""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tests import helpers as H


# ---- conversions -----------------------------------------------------------------
def test_f32_to_f16_soft_matches_numpy_on_random_bit_patterns():
    rng = np.random.default_rng(1)
    u = rng.integers(0, 2**32, size=1 << 16, dtype=np.uint64).astype(np.uint32)
    # add the rounding-boundary neighbourhood of every fp16 value
    h = np.arange(0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32).view(np.uint32)
    u = np.concatenate([u, h, h + 0x1000, h + 0x0fff, h + 0x1001, np.array([0x477fe000, 0x477fefff, 0x477ff000,
                                                                            0x33000000, 0x33000001, 0x32ffffff],
                                                                           np.uint32)])
    f = u.view(np.float32)
    L = orc.lib()
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    for i in range(0, f.size, 997):  # scalar ctypes calls: sample the array
        got = L.orc_f32_to_f16_soft(float(f[i])) if np.isfinite(f[i]) or np.isinf(f[i]) else 0x7fff
        if np.isnan(f[i]):
            continue
        assert got == want[i], (hex(u[i]), hex(got), hex(want[i]))
        assert L.orc_f32_to_f16(float(f[i])) == want[i]


def test_f16_to_f32_all_patterns():
    L = orc.lib()
    for hbits in list(range(0, 0x10000, 37)) + [0, 1, 0x3ff, 0x400, 0x7bff, 0x7c00, 0x8000, 0x8001, 0xfbff, 0xfc00]:
        want = np.array([hbits], np.uint16).view(np.float16).astype(np.float32)[0]
        if np.isnan(want):
            assert np.isnan(L.orc_f16_to_f32_soft(hbits))
            continue
        assert L.orc_f16_to_f32_soft(hbits) == want
        assert L.orc_f16_to_f32(hbits) == want


def test_bf16_to_fp16_all_65536_patterns_vs_numpy():
    src = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = orc.bf16_to_fp16(src)
    f = H.bf16_to_f32(src)
    with np.errstate(over="ignore", invalid="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    nan = np.isnan(f)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(got[nan] == 0x7fff)  # the reference's __float2half_rn canonical NaN


def test_bf16_to_fp16_is_exact_where_fp16_can_hold_bf16():
    # unbiased exponent in [-17, 15]: 8 significant bits fit fp16 normals and the top subnormal binades
    src = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    e = ((src >> 7) & 0xff).astype(np.int32) - 127
    sel = (e >= -17) & (e <= 15)
    got = orc.bf16_to_fp16(src[sel]).view(np.float16).astype(np.float32)
    assert np.array_equal(got, H.bf16_to_f32(src[sel]))
    # above 65504 -> Inf, far below 2^-25 -> signed zero
    big = H.f32_to_bf16(np.array([1e5, -1e5, 70000.0], np.float32))
    assert list(orc.bf16_to_fp16(big)) == [0x7c00, 0xfc00, 0x7c00]
    tiny = H.f32_to_bf16(np.array([1e-9, -1e-9], np.float32))
    assert list(orc.bf16_to_fp16(tiny)) == [0x0000, 0x8000]


# ---- embedding -----------------------------------------------------------------------
def test_embed_is_exact_row_copy():
    rng = np.random.default_rng(2)
    table = rng.integers(0, 65536, size=(50, 16), dtype=np.uint32).astype(np.uint16)
    ids = np.array([3, 49, 0, 3], np.int32)
    assert np.array_equal(orc.embed(table, ids), table[ids])


# ---- RMSNorm -----------------------------------------------------------------------------
@pytest.mark.parametrize("d", [256, 4096])
def test_rmsnorm_vs_float64(d):
    rng = np.random.default_rng(3)
    x = H.bits(rng.standard_normal((5, d)))
    g = H.bits(1.0 + 0.1 * rng.standard_normal(d))
    got = orc.rmsnorm(x, g)
    want = H.bits(H.rmsnorm_f64(x, g))
    assert H.ulp_diff(got, want).max() <= 1
    assert np.mean(got != want) < 0.01


def test_rmsnorm_unit_gain_gives_unit_mean_square_and_eps_matters():
    rng = np.random.default_rng(4)
    d = 4096
    x = H.bits(3.0 * rng.standard_normal((2, d)))
    one = H.bits(np.ones(d))
    y = H.f16(orc.rmsnorm(x, one))
    assert np.allclose(np.mean(y * y, axis=-1), 1.0, atol=2e-3)
    # tiny inputs: ss/d ~ 1e-6 < eps, so dropping eps (or using 1e-6) changes the result by > 2x
    xs = H.bits(1e-3 * rng.standard_normal((1, d)))
    got = H.f16(orc.rmsnorm(xs, one))
    want = H.rmsnorm_f64(xs, one, 1e-5)
    assert np.allclose(got, want, rtol=2e-3, atol=1e-4)
    assert not np.allclose(got, H.rmsnorm_f64(xs, one, 1e-6), rtol=0.2, atol=1e-4)


def test_rmsnorm_rejects_non_power_of_two():
    with pytest.raises(ValueError):
        orc.rmsnorm(np.zeros((1, 24), np.uint16), np.zeros(24, np.uint16))


# ---- residual add ------------------------------------------------------------------------------
def test_add_is_fp32_sum_rounded_once_to_fp16():
    """orc_add (reference add_norm, src/inference/inference.cu:377-390): fp16(float(x) + float(res)).
    Against numpy float32 on random values and on every pair from a set of edge patterns (signed
    zeros, subnormals, the largest finite value, infinities); the fp32 sum of two fp16 values is
    exact, so the result is the correctly rounded fp16 sum and float64 gives the same bits."""
    rng = np.random.default_rng(12)
    x = H.bits(rng.standard_normal(4099) * rng.choice([1e-4, 1.0, 300.0], 4099))
    r = H.bits(rng.standard_normal(4099) * rng.choice([1e-4, 1.0, 300.0], 4099))
    edge = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x03ff, 0x0400, 0x3c00, 0xbc00, 0x3c01, 0x7bff,
                     0xfbff, 0x7c00, 0xfc00, 0x1400, 0x6800], np.uint16)
    x = np.concatenate([x, np.repeat(edge, edge.size)])
    r = np.concatenate([r, np.tile(edge, edge.size)])
    got = orc.add(x, r)
    with np.errstate(over="ignore", invalid="ignore"):
        want32 = (x.view(np.float16).astype(np.float32) + r.view(np.float16).astype(np.float32)).astype(np.float16)
        want64 = (x.view(np.float16).astype(np.float64) + r.view(np.float16).astype(np.float64)).astype(np.float16)
    nan = np.isnan(want32)
    assert np.array_equal(got[~nan], want32.view(np.uint16)[~nan])
    assert np.array_equal(got[~nan], want64.view(np.uint16)[~nan])
    assert np.all(np.isnan(got[nan].view(np.float16)))       # Inf + -Inf
    assert orc.add(np.array([0x3c00], np.uint16), np.array([0x1000], np.uint16))[0] == 0x3c00  # 1 + half an ulp: tie to even
    assert orc.add(np.array([0x3c01], np.uint16), np.array([0x1000], np.uint16))[0] == 0x3c02  # odd mantissa: the tie rounds up


# ---- GEMM ----------------------------------------------------------------------------------
def test_linear_reference_gemm_test_operands_closed_form():
    # tests/gemm.cu:63-105 of the reference: X[8x8], Transform[4x8], A[i][j] = i*cols + j,
    # O = X . Transform^T  =>  O[i][c] = 512*i*c + 224*(i + c) + 140
    m, n, k = 8, 4, 8
    X = np.arange(m * k, dtype=np.float64).reshape(m, k)
    W = np.arange(n * k, dtype=np.float64).reshape(n, k)
    got = orc.linear(H.bits(X), H.bits(W))
    i, c = np.meshgrid(np.arange(m), np.arange(n), indexing="ij")
    want = 512.0 * i * c + 224.0 * (i + c) + 140.0
    assert got.shape == (m, n)  # [T, N]: a transposed output fails here
    assert np.array_equal(got, H.bits(want))  # fp16 rounding of the exact integers


def test_linear_vs_float64_non_square():
    rng = np.random.default_rng(5)
    T, N, K = 3, 24, 128
    x = H.bits(rng.standard_normal((T, K)))
    w = H.bits(0.02 * rng.standard_normal((N, K)))
    got = orc.linear(x, w)
    want = H.f16(x) @ H.f16(w).T
    assert H.ulp_diff(got, H.bits(want)).max() <= 1
    # T = 1 takes the other code path (interleaved row chains) and must give the same bits as T > 1
    assert np.array_equal(orc.linear(x[:1], w), got[:1])


def test_linear_accumulates_in_ascending_k_fp32():
    # 1 + 2^-24 + ... : ascending fp32 accumulation loses every small term, descending would not
    K = 64
    x = np.ones((1, K))
    w = np.full((8, K), 2.0 ** -13)
    w[:, 0] = 2048.0
    got = H.f16(orc.linear(H.bits(x), H.bits(w)))
    acc = np.float32(0)
    for kk in range(K):
        acc = np.float32(acc + np.float32(H.f16(H.bits(w))[0, kk]))
    assert got[0, 0] == np.float16(acc)


def test_swiglu_vs_float64_and_no_intermediate_rounding():
    rng = np.random.default_rng(6)
    T, N, K = 4, 16, 64
    x = H.bits(rng.standard_normal((T, K)))
    wg = H.bits(0.3 * rng.standard_normal((N, K)))
    wu = H.bits(0.3 * rng.standard_normal((N, K)))
    got = orc.linear_swiglu(x, wg, wu)
    g = H.f16(x) @ H.f16(wg).T
    u = H.f16(x) @ H.f16(wu).T
    want = H.silu(g) * u
    assert H.ulp_diff(got, H.bits(want)).max() <= 1
    # rounding gate and up to fp16 first (the reference's dead kernel_compute_swiglu) differs somewhere
    alt = H.silu(H.f16(H.bits(g))) * H.f16(H.bits(u))
    assert np.mean(got == H.bits(want)) > np.mean(got == H.bits(alt)) or np.array_equal(H.bits(want), H.bits(alt))


# ---- RoPE ---------------------------------------------------------------------------------------
def test_rope_position_zero_is_identity_and_norm_is_preserved():
    rng = np.random.default_rng(7)
    x = H.bits(rng.standard_normal((1, 8 * 128)))
    assert np.array_equal(orc.rope(x, 8, 128, pos0=0), x)
    y = H.f16(orc.rope(x, 8, 128, pos0=77)).reshape(-1, 2)
    assert np.allclose(np.linalg.norm(y, axis=1), np.linalg.norm(H.f16(x).reshape(-1, 2), axis=1), rtol=2e-3,
                       atol=1e-3)


def test_rope_pair_zero_rotates_by_pos_radians_and_pairs_are_adjacent():
    hd = 128
    x = np.zeros((1, hd))
    x[0, 0] = 1.0  # pair 0 = (x[0], x[1]) -- a half-split pairing would move x[64] instead
    y = H.f16(orc.rope(H.bits(x), 1, hd, pos0=3))
    assert np.allclose(y[0, :2], [np.cos(3.0), np.sin(3.0)], atol=1e-3)
    assert np.all(y[0, 2:] == 0)
    x[:] = 0
    x[0, 2 * 63] = 1.0  # last pair: angle = pos * theta^(-126/128)
    y = H.f16(orc.rope(H.bits(x), 1, hd, pos0=1000))
    a = 1000.0 * 500000.0 ** (-126.0 / 128.0)
    assert np.allclose(y[0, 126:128], [np.cos(a), np.sin(a)], atol=1e-3)


def test_rope_vs_float64_and_relative_position_property():
    rng = np.random.default_rng(8)
    T, Hh, hd = 6, 2, 32
    x = H.bits(rng.standard_normal((T, Hh * hd)))
    got = orc.rope(x, Hh, hd, pos0=40)
    assert H.ulp_diff(got, H.bits(H.rope_f64(x, Hh, hd, 40))).max() <= 1
    q = H.bits(rng.standard_normal((1, hd)))
    k = H.bits(rng.standard_normal((1, hd)))
    dots = []
    for m, n in [(5, 2), (105, 102), (1005, 1002)]:
        dots.append((H.f16(orc.rope(q, 1, hd, m)) @ H.f16(orc.rope(k, 1, hd, n)).T).item())
    assert np.allclose(dots, dots[0], atol=2e-2)


# ---- attention -----------------------------------------------------------------------------------------
def _qkv(rng, T, Hq, Hkv, hd, P=None):
    P = P or T
    return (H.bits(rng.standard_normal((T, Hq * hd))), H.bits(rng.standard_normal((P, Hkv * hd))),
            H.bits(rng.standard_normal((P, Hkv * hd))))


def test_attention_single_token_returns_v_of_mapped_kv_head():
    rng = np.random.default_rng(9)
    Hq, Hkv, hd = 8, 2, 32
    q, k, v = _qkv(rng, 1, Hq, Hkv, hd)
    out = orc.attention(q, k, v, 0, Hq, Hkv, hd).reshape(Hq, hd)
    vv = v.reshape(Hkv, hd)
    for h in range(Hq):
        assert np.array_equal(out[h], vv[h // 4])  # interleaved groups: kv = h / 4, not h % 2


def test_attention_uniform_keys_average_values_causally():
    rng = np.random.default_rng(10)
    T, Hq, Hkv, hd = 5, 4, 1, 32
    q, _, v = _qkv(rng, T, Hq, Hkv, hd)
    k = np.tile(H.bits(rng.standard_normal((1, hd))), (T, 1))
    out = H.f16(orc.attention(q, k, v, 0, Hq, Hkv, hd))
    vf = H.f16(v)
    for t in range(T):
        assert np.allclose(out[t, :hd], vf[:t + 1].mean(axis=0), atol=2e-3)


def test_attention_vs_float64_with_offset_and_materialized_form_bit_equal():
    rng = np.random.default_rng(11)
    T, Hq, Hkv, hd = 7, 8, 2, 32
    q, k, v = _qkv(rng, T, Hq, Hkv, hd)
    full = orc.attention(q, k, v, 0, Hq, Hkv, hd)
    assert H.mixed_err(full, H.bits(H.attention_f64(q, k, v, 0, Hq, Hkv, hd))) < 2e-3
    # the reference's own three-kernel schedule gives the same bits
    assert np.array_equal(orc.attention_materialized(q, k, v, Hq, Hkv, hd), full)
    # last two rows alone, with the first five positions as cache
    part = orc.attention(q[5:], k, v, 5, Hq, Hkv, hd)
    assert np.array_equal(part, full[5:])
    # scale is 1/sqrt(head_dim): with 1/sqrt(n_heads) (tests/llama3.py:65) the result differs
    qs = H.bits(H.f16(q) * np.sqrt(hd) / np.sqrt(Hq))
    assert H.mixed_err(orc.attention(qs, k, v, 0, Hq, Hkv, hd), full) > 1e-2


# ---- argmax ----------------------------------------------------------------------------------------------
def test_argmax_ties_zero_signs_nan():
    b = H.bits
    assert orc.argmax_f16(b([1.0, 3.0, 3.0, 2.0])) == 1
    assert orc.argmax_f16(b([-0.0, 0.0, -1.0])) == 0
    assert orc.argmax_f16(b([0.0, -0.0])) == 0
    v = b([1.0, 2.0, 0.5])
    v[1] = 0x7e00
    assert orc.argmax_f16(v) == 0
    assert orc.argmax_f16(np.array([0x7e00, 0xfe00], np.uint16)) == 0
    assert orc.argmax_f16(b([-np.inf, -5.0])) == 1
    rng = np.random.default_rng(12)
    x = b(rng.standard_normal(5000))
    assert orc.argmax_f16(x) == int(np.argmax(H.f16(x)))
