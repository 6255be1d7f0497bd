"""Writes tests/golden/tiny_seed1234.json: the tiny-configuration prompt, the 32
greedy tokens and bit-sum checksums of the per-layer hidden states and logits,
all from the ORC_REF16 oracle on the seeded weights.  The reference itself
holds no golden vectors for this path and cannot run here (CUDA only), so the
fixture pins the oracle build across machines rather than the reference.

    python tests/golden/make_tiny_fixture.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import __graft_entry__ as ge  # noqa: E402
from oracle import pyoracle as orc  # noqa: E402
from tests import helpers as H  # noqa: E402

SEED, N_PROMPT, N_DECODE = 1234, 16, 32

pkg = ge.load_package()
cfg = pkg.engine.config("tiny")
model = pkg.engine.Model.seeded(cfg, SEED)
w = H.oracle_weights(model)
prompt = pkg.engine.seeded_tokens(SEED, N_PROMPT, cfg.vocab)
m = orc.Model(H.cfg_dict(cfg), w, orc.ORC_REF16)
tok, hid, logits = m.forward(prompt, want_hidden=True)
toks = [tok]
for _ in range(N_DECODE - 1):
    tok, _, _ = m.forward([tok])
    toks.append(tok)
out = {
    "config": H.cfg_dict(cfg), "seed": SEED, "prompt": [int(t) for t in prompt], "tokens": [int(t) for t in toks],
    "hidden_bit_sums": [int(hid[l].astype(np.uint64).sum()) for l in range(cfg.n_layers)],
    "logits_bit_sum": int(logits.astype(np.uint64).sum()),
}
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tiny_seed1234.json")
json.dump(out, open(path, "w"), indent=1)
print("wrote", path, out["tokens"][:8])
