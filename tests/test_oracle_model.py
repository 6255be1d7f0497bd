"""Whole-model checks of the oracle on the CPU-runnable tiny configuration
(2 layers, d 256, 8/2 heads, head_dim 32, FFN 768, vocab 4096; prompt of 16
seeded ids, 32 greedy tokens): KV cache == the reference's full recompute bit
for bit, ORC_REF16 vs ORC_FP32 inside 2e-2, and the committed golden fixture."""
import json
import os

import numpy as np
import pytest

from oracle import pyoracle as orc
from tests import helpers as H

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_seed1234.json")
SEED, N_PROMPT, N_DECODE = 1234, 16, 32


def _setup(pkg):
    cfg = pkg.engine.config("tiny")
    model = pkg.engine.Model.seeded(cfg, SEED)
    w = H.oracle_weights(model)
    model.close()
    prompt = pkg.engine.seeded_tokens(SEED, N_PROMPT, cfg.vocab)
    return cfg, H.cfg_dict(cfg), w, prompt


def test_cache_equals_full_recompute_bit_for_bit(pkg):
    cfg, cd, w, prompt = _setup(pkg)
    m = orc.Model(cd, w, orc.ORC_REF16)
    tok, hid, logits = m.forward(prompt, want_hidden=True)
    tok_r, hid_r, logits_r = orc.forward_recompute(cd, w, prompt, want_hidden=True)
    assert tok == tok_r and np.array_equal(hid, hid_r) and np.array_equal(logits, logits_r)
    # three cached decode steps vs recompute of the grown sequence
    seq = list(prompt) + [tok]
    for _ in range(3):
        t, h1, lg = m.forward([seq[-1]], want_hidden=True)
        t_r, h_r, lg_r = orc.forward_recompute(cd, w, seq, want_hidden=True)
        assert t == t_r and np.array_equal(lg, lg_r)
        assert np.array_equal(h1[:, 0, :], h_r[:, -1, :])
        seq.append(t)
    # a split prompt (prefill in two chunks) gives the same bits as one chunk
    m2 = orc.Model(cd, w, orc.ORC_REF16)
    m2.forward(prompt[:9])
    tok2, _, logits2 = m2.forward(prompt[9:])
    assert tok2 == tok and np.array_equal(logits2, logits)


def test_ref16_and_fp32_agree_within_tolerance(pkg):
    cfg, cd, w, prompt = _setup(pkg)
    a = orc.Model(cd, w, orc.ORC_REF16)
    b = orc.Model(cd, w, orc.ORC_FP32)
    ta, ha, la = a.forward(prompt, want_hidden=True)
    tb, hb, lb = b.forward(prompt, want_hidden=True)
    assert H.mixed_err(ha, hb) < H.TOL and H.mixed_err(la, lb) < H.TOL
    assert ta == tb


def test_reversed_order_mode_is_a_reordering_only(pkg):
    """ORC_REF16_REV sums every projection over k downwards: close to ORC_REF16 (same terms), not
    identical (fp32 addition is not associative), and the switch does not leak into later models."""
    cfg, cd, w, prompt = _setup(pkg)
    a = orc.Model(cd, w, orc.ORC_REF16)
    r = orc.Model(cd, w, orc.ORC_REF16_REV)
    ta, ha, la = a.forward(prompt, want_hidden=True)
    tr, hr, lr = r.forward(prompt, want_hidden=True)
    assert H.mixed_err(ha, hr) < H.TOL and H.mixed_err(la, lr) < H.TOL
    assert not np.array_equal(ha, hr)
    assert ta == tr
    # the mode must not leak into later ORC_REF16 models
    a2 = orc.Model(cd, w, orc.ORC_REF16)
    _, ha2, _ = a2.forward(prompt, want_hidden=True)
    assert np.array_equal(ha, ha2)


def test_golden_fixture(pkg):
    """tests/golden/tiny_seed1234.json was written by tests/golden/make_tiny_fixture.py
    from this oracle; it travels to the GPU box and pins the oracle build there
    (same tokens, same hidden-state checksums)."""
    cfg, cd, w, prompt = _setup(pkg)
    g = json.load(open(GOLDEN))
    assert g["prompt"] == [int(t) for t in prompt]
    m = orc.Model(cd, w, orc.ORC_REF16)
    tok, hid, logits = m.forward(prompt, want_hidden=True)
    toks = [tok]
    for _ in range(N_DECODE - 1):
        tok, _, _ = m.forward([tok])
        toks.append(tok)
    assert toks == g["tokens"]
    assert [int(hid[l].astype(np.uint64).sum()) for l in range(cfg.n_layers)] == g["hidden_bit_sums"]
    assert int(logits.astype(np.uint64).sum()) == g["logits_bit_sum"]


# ---- the wiring of the whole model, against an independent float64 forward ------------------
def _distinct_gain_weights(w, cfg, seed):
    """The seeded tiny model has unit norm gains; give every norm its own random gains so that a
    norm applied with the wrong gains (or not at all) changes the result."""
    rng = np.random.default_rng(seed)
    w = dict(w)
    gain = lambda: H.bits(rng.uniform(0.5, 1.5, cfg.d_model))
    w["input_ln"] = [gain() for _ in range(cfg.n_layers)]
    w["post_ln"] = [gain() for _ in range(cfg.n_layers)]
    w["norm"] = gain()
    return w


def _rel_err(a, b):
    return float(np.max(np.abs(a - b) / (1.0 + np.abs(b))))


def test_model_wiring_vs_independent_float64_forward(pkg):
    """orc_model_forward (ORC_FP32: the same graph as ORC_REF16 without intermediate rounding) against
    tests/helpers.model_forward_f64, which is written from the reference driver
    (src/inference/inference.cu:149-193, LM head on the last row :1014) out of numpy closed forms and
    shares no code with oracle.c.  Per-layer hidden states and logits within 1e-3, same argmax; then
    ORC_REF16 within the model tolerance of the same float64 result."""
    cfg, cd, w, prompt = _setup(pkg)
    w = _distinct_gain_weights(w, cfg, 7)
    hid64, lg64 = H.model_forward_f64(cd, w, [int(t) for t in prompt])
    m = orc.Model(cd, w, orc.ORC_FP32)
    tok, hid, lg = m.forward(prompt, want_hidden=True)
    for l in range(cfg.n_layers):
        assert _rel_err(H.f16(hid[l]), hid64[l]) < 1e-3, l   # fp16 export of an fp32 state: 2^-11 relative
    assert _rel_err(H.f16(lg), lg64) < 1e-3
    assert tok == int(np.argmax(lg64))
    m16 = orc.Model(cd, w, orc.ORC_REF16)
    tok16, hid16, lg16 = m16.forward(prompt, want_hidden=True)
    assert max(_rel_err(H.f16(hid16[l]), hid64[l]) for l in range(cfg.n_layers)) < H.TOL
    assert _rel_err(H.f16(lg16), lg64) < H.TOL
    assert tok16 == int(np.argmax(lg64))
    # decode steps through the KV cache against the float64 forward of the grown sequence
    seq = [int(t) for t in prompt] + [tok]
    for _ in range(3):
        t, h1, lg = m.forward([seq[-1]], want_hidden=True)
        hid64, lg64 = H.model_forward_f64(cd, w, seq)
        assert _rel_err(H.f16(h1[:, 0, :]), hid64[:, -1, :]) < 1e-3
        assert _rel_err(H.f16(lg), lg64) < 1e-3 and t == int(np.argmax(lg64))
        seq.append(t)


@pytest.mark.parametrize("mistake", ["swap_norm_gains", "residual_after_norm", "no_final_norm",
                                     "swap_gate_up", "no_rope"])
def test_wiring_check_is_sensitive_to_plausible_mistakes(pkg, mistake):
    """The comparison above would fail for each plausible wiring mistake: the float64 forward with the
    mistake built in is far outside 1e-3 of the oracle."""
    cfg, cd, w, prompt = _setup(pkg)
    w = _distinct_gain_weights(w, cfg, 7)
    m = orc.Model(cd, w, orc.ORC_FP32)
    _, hid, lg = m.forward(prompt, want_hidden=True)
    hid_bad, lg_bad = H.model_forward_f64(cd, w, [int(t) for t in prompt], mutate=mistake)
    worst = max(_rel_err(H.f16(lg), lg_bad), max(_rel_err(H.f16(hid[l]), hid_bad[l]) for l in range(cfg.n_layers)))
    assert worst > 1e-2, (mistake, worst)


def test_single_layer_model_wiring(pkg):
    """One layer, distinct gains: nothing can hide behind a second layer."""
    cfg, cd, w, prompt = _setup(pkg)
    w = _distinct_gain_weights(w, cfg, 11)
    cd1 = dict(cd, n_layers=1)
    w1 = {k: (v[:1] if isinstance(v, list) else v) for k, v in w.items()}
    hid64, lg64 = H.model_forward_f64(cd1, w1, [int(t) for t in prompt])
    tok, hid, lg = orc.Model(cd1, w1, orc.ORC_FP32).forward(prompt, want_hidden=True)
    assert _rel_err(H.f16(hid[0]), hid64[0]) < 1e-3 and _rel_err(H.f16(lg), lg64) < 1e-3
    assert tok == int(np.argmax(lg64))
