"""The decode step's hand-over launches (attention and output projection in one launch, the projection's
workgroups waiting for the attention's result inside the kernel): a wait that gives up must cost a redone
step, not the process; engines that step at the same time on their own streams must not disturb each
other's waits."""
import threading

import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def _model(gpu, which, seed, max_pos):
    cfg = gpu.engine.config("tiny", max_pos=max_pos) if which == "tiny" else gpu.engine.config("8b", n_layers=2, max_pos=max_pos)
    return cfg, gpu.engine.Model.seeded(cfg, seed).to_device()


@pytest.mark.parametrize("which,n_prompt", [("tiny", 20), ("tiny", 505), ("8b", 9)])
def test_a_counted_timeout_redoes_the_step(gpu, which, n_prompt):
    """A step that reports a wait that gave up (the count is set from the host before the step: every kernel
    runs to its normal end) is redone with one launch per operation: same ids and logits as an engine that
    never used the hand-over launches, through llama3_decode, llama3_generate and a one-token prompt pass;
    the cache keeps the plain form afterwards and can be put back."""
    cfg, model = _model(gpu, which, 91, 1024)
    prompt = gpu.engine.seeded_tokens(91, n_prompt, cfg.vocab)
    ref = gpu.engine.Engine(model, cfg, use_graph=False)
    ref.set_handover(False)
    assert ref.handover_stats() == (0, 0, False)
    want, _ = ref.generate(prompt, 20)     # the second tiny case crosses position 512: both hand-over forms
    want = [int(t) for t in want]
    for use_graph in (True, False):
        eng = gpu.engine.Engine(model, cfg, use_graph=use_graph)
        assert eng.handover_stats() == (0, 0, True)
        # llama3_decode: the marked step is the third
        t, _ = eng.prefill(prompt)
        got = [t]
        ref.reset()
        t_r, _ = ref.prefill(prompt)
        for step in range(6):
            if step == 2:
                eng.mark_handover_timeout()
            t, _ = eng.decode(t)
            t_r, _ = ref.decode(t_r)
            got.append(t)
            assert np.array_equal(eng.logits(), ref.logits()), (use_graph, step)
            assert eng.handover_stats() == ((0, 0, True) if step < 2 else (1, 1, False)), step
        assert got == want[:7], (use_graph, got, want[:7])
        # back into the hand-over form; llama3_generate with a mark: its run of steps is redone as a whole
        eng.set_handover(True)
        eng.reset()
        eng.mark_handover_timeout()
        toks, _ = eng.generate(prompt, 20)
        assert [int(x) for x in toks] == want, use_graph
        assert eng.handover_stats() == (2, 2, False)
        # the position on the device and the host agree after the redo: further steps continue the sequence
        t_more, _ = eng.decode(int(toks[-1]))
        ref.reset()
        ref.generate(prompt, 20)
        t_ref, _ = ref.decode(want[-1])
        assert t_more == t_ref
        eng.close()
    ref.close()
    model.close()


@pytest.mark.parametrize("which", ["tiny", "8b"])
def test_waits_that_really_give_up_cost_a_redo_not_the_result(gpu, which):
    """With the bound of the wait at zero polling rounds a projection workgroup gives up whenever the
    attention's result is not there at its first look (whether that happens depends on timing): every kernel
    still ends normally, the host redoes what was affected, and the ids are those of the plain form."""
    cfg, model = _model(gpu, which, 92, 256)
    prompt = gpu.engine.seeded_tokens(92, 17, cfg.vocab)
    ref = gpu.engine.Engine(model, cfg, use_graph=False)
    ref.set_handover(False)
    want, _ = ref.generate(prompt, 24)
    eng = gpu.engine.Engine(model, cfg)
    eng.set_handover(True, spin_limit=0)
    got, _ = eng.generate(prompt, 24)
    timeouts, recoveries, active = eng.handover_stats()
    say(which, "waits that gave up:", timeouts, "redone:", recoveries, "hand-over still on:", active)
    assert [int(x) for x in got] == [int(x) for x in want]
    assert (timeouts == 0) == (recoveries == 0) and active == (recoveries == 0)
    assert np.array_equal(eng.logits(), ref.logits())
    eng.close()
    ref.close()
    model.close()


@pytest.mark.parametrize("which,n_prompt,n_decode", [("tiny", 30, 120), ("tiny", 500, 60), ("8b", 40, 100)])
def test_two_engines_stepping_at_once_on_their_own_streams(gpu, which, n_prompt, n_decode):
    """Two caches of one model, each on its own stream, driven from two host threads at the same time (graph
    replays of the hand-over launches back to back on both streams): no wait gives up, nothing is redone, and
    each engine produces the ids it produces alone."""
    cfg, model = _model(gpu, which, 93, 1024)
    prompts = [gpu.engine.seeded_tokens(200 + i, n_prompt + 7 * i, cfg.vocab) for i in range(2)]
    alone = []
    for p in prompts:
        e = gpu.engine.Engine(model, cfg)
        t, _ = e.generate(p, n_decode)
        alone.append([int(x) for x in t])
        e.close()
    engines = [gpu.engine.Engine(model, cfg) for _ in range(2)]
    for e, p in zip(engines, prompts):      # capture the graphs before the concurrent part
        e.generate(p, 3)
        e.reset()
    results, errors = [None, None], []
    start = threading.Barrier(2)

    def run(i):
        try:
            start.wait()
            out = []
            for rep in range(3):
                engines[i].reset()
                t, _ = engines[i].generate(prompts[i], n_decode)
                out.append([int(x) for x in t])
            results[i] = out
        except Exception as exc:  # noqa: BLE001
            errors.append((i, repr(exc)))

    threads = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    for i in range(2):
        assert results[i] is not None
        for rep, r in enumerate(results[i]):
            assert r == alone[i], (i, rep)
        assert engines[i].handover_stats() == (0, 0, True), engines[i].handover_stats()
        engines[i].close()
    model.close()


def test_handover_ops_with_a_zero_wait_bound_end_normally(gpu):
    """The kernel-level view of a wait that gives up: llm_attn_decode_rope_oproj and its long-context form with
    spin_limit 0 return, count what they gave up on, and the same buffers serve a correct launch after they are
    filled again (the wrapper starts every call from freshly armed buffers)."""
    Hq, Hkv, hd, N = 32, 8, 128, 4096
    for pos, max_pos, long_form in ((200, 512, False), (700, 1024, True)):
        rng = np.random.default_rng(pos)
        qd, kvd = Hq * hd, Hkv * hd
        qkv = H.bits(rng.standard_normal((1, qd + 2 * kvd)))
        k_old, v_old = H.bits(rng.standard_normal((pos, kvd))), H.bits(rng.standard_normal((pos, kvd)))
        kc, vc = gpu.ops.kv_layout(k_old, v_old, Hkv, hd, max_pos)
        w = H.bits(0.05 * rng.standard_normal((N, qd)))
        a0, o0, _, _, t0 = gpu.ops.attn_decode_rope_oproj(qkv, kc, vc, pos, Hq, Hkv, hd, w, long_form=long_form, spin_limit=0)
        a1, o1, _, _, t1 = gpu.ops.attn_decode_rope_oproj(qkv, kc, vc, pos, Hq, Hkv, hd, w, long_form=long_form)
        say("zero wait bound at position", pos, "gave up:", t0)
        assert t1 == 0 and t0 >= 0
        assert np.array_equal(a0, a1)            # the attention itself never waits
        if t0 == 0:
            assert np.array_equal(o0, o1)
