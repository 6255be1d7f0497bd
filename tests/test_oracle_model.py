"""Whole-model checks of the oracle on the CPU-runnable tiny configuration
(2 layers, d 256, 8/2 heads, head_dim 32, FFN 768, vocab 4096; prompt of 16
seeded ids, 32 greedy tokens): KV cache == the reference's full recompute bit
for bit, ORC_REF16 vs ORC_FP32 inside 2e-2, and the committed golden fixture."""
import json
import os

import numpy as np

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
