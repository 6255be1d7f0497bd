"""The two full-size workloads at all 32 layers of LLaMA3-8B, checked through properties that need no
CPU oracle run (which would take hours at this size): a captured decode graph, plain launches and the
step-by-step API produce the same ids; a prompt fed in one pass and in chunks leaves the same state; decode
across positions 8192..8704 is the same with and without graphs.  Parity with the oracle is established at
sizes the oracle can reach in tests/test_gpu_model.py and tests/test_gpu_ops.py; these tests carry it to
the full shapes."""
import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def model_8b(gpu):
    cfg = gpu.engine.config("8b", max_pos=8704)
    say("full size: seeded 8B weights (16 GB) ...")
    model = gpu.engine.Model.seeded(cfg, 4242).to_device()
    yield cfg, model
    model.close()


def test_prompt_128_then_256_steps_graph_plain_and_stepwise_agree(gpu, model_8b):
    cfg, model = model_8b
    prompt = gpu.engine.seeded_tokens(41, 128, cfg.vocab)
    eng = gpu.engine.Engine(model, cfg, use_graph=True)
    a, st = eng.generate(prompt, 256)
    assert eng.pos == 128 + 255
    eng.reset()
    b, _ = eng.generate(prompt, 256)  # replay of the graphs captured by the first run
    eng.close()
    plain = gpu.engine.Engine(model, cfg, use_graph=False)
    c, _ = plain.generate(prompt, 256)
    plain.reset()
    tok, _ = plain.prefill(prompt)
    d = [tok]
    for _ in range(255):
        tok, _ = plain.decode(d[-1])
        d.append(tok)
    plain.close()
    say("prompt 128 + 256 steps: first ids", list(a[:8]), "decode ms/token", st.decode_ms / max(1, st.n_decode_steps))
    assert list(a) == list(b), "graph replay differs from the capturing run"
    assert list(a) == list(c), "captured graph differs from plain launches"
    assert list(a) == d, "generate() differs from prefill() + decode() per token"
    assert len(set(a.tolist())) > 16  # a degenerate constant sequence would make the equalities empty


def test_prompt_8192_then_512_steps_graph_equals_plain_and_chunked_prompt(gpu, model_8b):
    cfg, model = model_8b
    prompt = gpu.engine.seeded_tokens(42, 8192, cfg.vocab)
    eng = gpu.engine.Engine(model, cfg, use_graph=True)
    a, st = eng.generate(prompt, 512)  # one 8192-row pass, then 511 graph replays at positions 8192..8702
    assert eng.pos == 8192 + 511
    eng.close()
    plain = gpu.engine.Engine(model, cfg, use_graph=False)
    b, _ = plain.generate(prompt, 512)
    say("prompt 8192 + 512 steps: first ids", list(a[:8]), "prompt pass ms", st.prefill_ms,
        "decode ms/token", st.decode_ms / max(1, st.n_decode_steps))
    assert list(a) == list(b), "captured graph differs from plain launches at positions 8192.."
    assert len(set(a.tolist())) > 16

    # the same prompt in one pass and in two unequal chunks: same state within the model tolerance
    plain.reset()
    t_full, h_full = plain.prefill(prompt, want_hidden=True)
    lg_full = plain.logits()
    assert t_full == a[0]
    plain.reset()
    plain.prefill(prompt[:5000])
    t_part, h_part = plain.prefill(prompt[5000:], want_hidden=True)
    lg_part = plain.logits()
    rows = np.r_[0:128, 1500:1628, 3064:3192]  # of the second chunk: its start, middle and end
    errs = [H.mixed_err(h_part[l][rows], h_full[l][5000 + rows]) for l in range(cfg.n_layers)]
    e_lg = H.mixed_err(lg_part, lg_full)
    same = [bool(np.array_equal(h_part[l], h_full[l][5000:])) for l in (0, cfg.n_layers - 1)]
    say("8192 prompt, one pass vs 5000+3192: hidden err per layer", np.round(errs, 5).tolist(), "logits err", e_lg,
        "first / last layer bit-identical:", same, "ids", t_full, t_part)
    assert max(errs) <= H.TOL and e_lg <= H.TOL
    assert H.same_pick_or_near_tie(lg_part, lg_full, t_part, t_full)
    plain.close()
