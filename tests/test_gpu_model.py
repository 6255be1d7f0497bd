"""Whole-model parity of the HIP engine against the CPU oracle on identical
seeded weights and prompts: bit-exact weight conversion, per-layer hidden
states and logits inside 2e-2, identical greedy tokens, graph replay equal to
plain launches, the reference-shaped inference() call, chunked prompts."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from oracle import pyoracle as orc
from tests import helpers as H

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_seed1234.json")


def say(*a):
    print(*a, flush=True)


def test_tiny_model_matches_oracle_and_golden_fixture(gpu):
    cfg = gpu.engine.config("tiny")
    r = H.run_model_parity(gpu, cfg, seed=1234, n_prompt=16, n_decode=32)
    say({k: v for k, v in r.items() if k not in ("top2_gaps",)})
    assert r["convert_exact"]
    assert r["hidden_max_err"] <= H.TOL and r["logits_max_err"] <= H.TOL
    assert r["argmax_matches_own_logits"]
    assert r["tokens_gpu"] == r["tokens_oracle"]
    g = json.load(open(GOLDEN))
    assert r["tokens_gpu"] == g["tokens"]


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_tiny_model_other_seeds_and_no_graph(gpu, seed):
    cfg = gpu.engine.config("tiny", max_pos=128)
    r = H.run_model_parity(gpu, cfg, seed=seed, n_prompt=40, n_decode=32, use_graph=(seed != 2))
    say(seed, r["hidden_max_err"], r["logits_max_err"], r["tokens_gpu"][:8], min(r["top2_gaps"]))
    assert r["convert_exact"] and r["hidden_max_err"] <= H.TOL and r["logits_max_err"] <= H.TOL
    assert r["tokens_gpu"] == r["tokens_oracle"]


def _tiny_engine(gpu, seed=5, max_pos=128, use_graph=True):
    cfg = gpu.engine.config("tiny", max_pos=max_pos)
    model = gpu.engine.Model.seeded(cfg, seed).to_device()
    return cfg, model, gpu.engine.Engine(model, cfg, use_graph=use_graph)


def test_graph_replay_equals_plain_launches_and_stepwise_api(gpu):
    cfg, model, eng = _tiny_engine(gpu, use_graph=True)
    prompt = gpu.engine.seeded_tokens(5, 20, cfg.vocab)
    a, _ = eng.generate(prompt, 40)
    eng.reset()
    b, _ = eng.generate(prompt, 40)  # second run replays the captured graph after other work
    eng.close()
    eng2 = gpu.engine.Engine(model, cfg, use_graph=False)
    c, _ = eng2.generate(prompt, 40)
    eng2.reset()
    tok, _ = eng2.prefill(prompt)
    d = [tok]
    for _ in range(39):
        tok, _ = eng2.decode(d[-1])
        d.append(tok)
    eng2.close()
    model.close()
    assert list(a) == list(b) == list(c) == d


def test_reference_shaped_inference_call(gpu):
    """inference(model, X, d_tokens, h_tokens, cache) with tokens[0] = n + 1, as src/main.cu:112-123 drives it."""
    cfg, model, eng = _tiny_engine(gpu)
    prompt = [int(t) for t in gpu.engine.seeded_tokens(5, 12, cfg.vocab)]
    seq = list(prompt)
    for _ in range(6):
        seq.append(eng.inference(seq))
    assert eng.pos == len(seq) - 1
    ref, _ = gpu.engine.Engine(model, cfg).generate(np.array(prompt, np.int32), 6)
    assert seq[len(prompt):] == [int(t) for t in ref]
    # a new, unrelated prompt resets the cache (the reference recomputes everything anyway)
    other = [int(t) for t in gpu.engine.seeded_tokens(6, 9, cfg.vocab)]
    t1 = eng.inference(other)
    eng.reset()
    t2, _ = eng.prefill(np.array(other, np.int32))
    assert t1 == t2
    # the reference's own next-token rule: host sampler over the fp16 logits, libc rand() never seeded
    libc = C.CDLL("libc.so.6")
    eng.set_sampling(True)
    libc.srand(1)
    rnd = orc.Rand(1)
    seq = list(prompt)
    for _ in range(6):
        tok = eng.inference(seq)
        assert tok == orc.sample(eng.logits(), rnd)
        seq.append(tok)
    eng.set_sampling(False)
    eng.close()
    model.close()


def test_inference_call_leaves_logits_on_the_host_and_mirrors_d_tokens(gpu):
    """After inference() returns, CudaCache.h_token_probdist holds the step's fp16 logits (as after the
    reference's compute_lm_head, inference.cu:1021-1026) and the caller's d_tokens array holds the
    token list; the greedy id is the argmax of exactly those logits."""
    cfg, model, eng = _tiny_engine(gpu)
    d_tokens = gpu.capi.DevBuf((2048,), np.int32)
    d_tokens.zero()
    seq = [int(t) for t in gpu.engine.seeded_tokens(9, 10, cfg.vocab)]
    for step in range(5):
        tok = eng.inference(seq, d_tokens)
        lg = eng.host_logits()
        assert np.array_equal(lg, eng.logits())
        assert tok == orc.argmax_f16(lg)
        mirror = d_tokens.download()
        assert mirror[0] == len(seq) + 1 and list(mirror[1:len(seq) + 1]) == seq
        # a caller that does not follow the greedy id (a sampler): the step must use the caller's id
        seq.append(tok if step % 2 == 0 else (tok + 1) % cfg.vocab)
    # same sequence through the stepwise API on a fresh cache
    eng2 = gpu.engine.Engine(model, cfg, use_graph=False)
    t2, _ = eng2.prefill(np.array(seq[:-1], np.int32))
    assert t2 == tok
    eng.close()
    eng2.close()
    model.close()


def test_two_caches_with_different_vocabularies_sample_independently(gpu):
    """Sampler settings live in the cache: two live caches of different vocabulary sizes, inference() with
    the reference's sampler on both, interleaved; each draw equals the oracle's on that cache's logits."""
    cfg_a = gpu.engine.config("tiny", max_pos=64)
    cfg_b = gpu.engine.config("tiny", max_pos=64, vocab=1024)
    model_a = gpu.engine.Model.seeded(cfg_a, 31).to_device()
    model_b = gpu.engine.Model.seeded(cfg_b, 32).to_device()
    eng_a, eng_b = gpu.engine.Engine(model_a, cfg_a), gpu.engine.Engine(model_b, cfg_b)
    eng_b.sampler_config(1.1, 20, 0.8)
    eng_a.set_sampling(True)
    eng_b.set_sampling(True)
    libc = C.CDLL("libc.so.6")
    libc.srand(5)
    rnd = orc.Rand(5)
    seq_a = [int(t) for t in gpu.engine.seeded_tokens(1, 7, cfg_a.vocab)]
    seq_b = [int(t) for t in gpu.engine.seeded_tokens(2, 9, cfg_b.vocab)]
    for _ in range(6):
        ta = eng_a.inference(seq_a)
        assert ta == orc.sample(eng_a.host_logits(), rnd)
        seq_a.append(ta)
        tb = eng_b.inference(seq_b)
        assert 0 <= tb < cfg_b.vocab and tb == orc.sample(eng_b.host_logits(), rnd, 1.1, 20, 0.8)
        seq_b.append(tb)
    libc.srand(1)
    for e in (eng_a, eng_b):
        e.close()
    for m in (model_a, model_b):
        m.close()


def test_cache_follows_a_change_of_model(gpu):
    """A cache whose decode graph was captured with one model is then driven with another model of the
    same configuration: the graph is captured again, the ids are those of a fresh cache on that model."""
    cfg = gpu.engine.config("tiny", max_pos=64)
    m1 = gpu.engine.Model.seeded(cfg, 41).to_device()
    m2 = gpu.engine.Model.seeded(cfg, 42).to_device()
    prompt = gpu.engine.seeded_tokens(3, 8, cfg.vocab)
    eng = gpu.engine.Engine(m1, cfg, use_graph=True)
    a1, _ = eng.generate(prompt, 6)
    eng.reset()
    eng.model = m2
    a2, _ = eng.generate(prompt, 6)
    ref = gpu.engine.Engine(m2, cfg, use_graph=False)
    b2, _ = ref.generate(prompt, 6)
    assert list(a2) == list(b2) and list(a1) != list(a2)
    eng.close()
    ref.close()
    m1.close()
    m2.close()


def test_decode_across_the_long_context_attention_switch(gpu):
    """Greedy decoding from position 500 to 560 changes attention kernels at 512 cached positions (one
    launch before, span + merge launches after) and graphs with them: same ids with and without graphs,
    same as stepping through the API, and the oracle agrees on hidden states on both sides."""
    cfg = gpu.engine.config("tiny", max_pos=1024)
    model = gpu.engine.Model.seeded(cfg, 21)
    w = H.oracle_weights(model)
    model.to_device()
    prompt = gpu.engine.seeded_tokens(21, 500, cfg.vocab)
    eng = gpu.engine.Engine(model, cfg, use_graph=True)
    a, _ = eng.generate(prompt, 60)
    eng.reset()
    b, _ = eng.generate(prompt, 60)
    eng.close()
    eng2 = gpu.engine.Engine(model, cfg, use_graph=False)
    c, _ = eng2.generate(prompt, 60)
    assert list(a) == list(b) == list(c)
    # step API with hidden states against the oracle, fed with the engine's own ids
    o = orc.Model(H.cfg_dict(cfg), w, orc.ORC_REF16)
    eng2.reset()
    tok, _ = eng2.prefill(prompt)
    tok_o, _, _ = o.forward(prompt)
    assert tok == tok_o == a[0]
    worst = 0.0
    for i in range(1, 40):
        t_g, h_g = eng2.decode(int(a[i - 1]), want_hidden=True)
        t_o, h_o, lg_o = o.forward([int(a[i - 1])], want_hidden=True)
        worst = max(worst, H.mixed_err(h_g, h_o), H.mixed_err(eng2.logits(), lg_o))
        assert t_g == a[i]
    say("long-context switch: worst err", worst)
    assert worst <= H.TOL
    o.close()
    eng2.close()
    model.close()


def _all_device_tensors(model, cfg):
    h = model.handle.contents
    out = [model.device_fp16(h.embed_tokens), model.device_fp16(h.lm_head), model.device_fp16(h.norm)]
    for l in range(cfg.n_layers):
        L = h.layers[l].contents
        for slot in ("input_layernorm", "mlp_down_proj", "mlp_gate_proj", "mlp_up_proj", "post_attention_layernorm",
                     "self_attn_k_proj", "self_attn_o_proj", "self_attn_q_proj", "self_attn_v_proj"):
            out.append(model.device_fp16(getattr(L, slot)))
    return out


@pytest.mark.parametrize("which", ["tiny", "8b-2-layers"])
def test_streaming_load_equals_load_then_to_cuda(gpu, tmp_path, which):
    """load_safetensor_weights_streaming() leaves the same fp16 bits on the device as the reference's
    two steps; the 8B shapes make the embedding and LM head span 16 staging chunks each."""
    import time
    cfg = gpu.engine.config("tiny") if which == "tiny" else gpu.engine.config("8b", n_layers=2, max_pos=64)
    path = str(tmp_path / "model.safetensors")
    assert gpu.lib().seeded_write_safetensors(C.byref(cfg), 31, path.encode()) == 0
    t0 = time.time()
    a = gpu.engine.Model.from_files(cfg, [path]).to_device()
    t1 = time.time()
    b = gpu.engine.Model.from_files_streaming(cfg, [path])
    t2 = time.time()
    say("%s: %.1f MB file, load + to_cuda %.2f s, streaming %.2f s" % (which, os.path.getsize(path) / 1e6, t1 - t0, t2 - t1))
    for x, y in zip(_all_device_tensors(a, cfg), _all_device_tensors(b, cfg)):
        assert x.shape == y.shape and np.array_equal(x, y)
    a.close()
    b.close()
    os.remove(path)


def test_driver_chat_turn_with_tokenizer(gpu, tmp_path):
    """llama3_main --tokenizer --text: the reference's chat turn (template, trie tokenizer, inference() per
    token, decode table) end to end on the tiny model with a synthetic tokenizer.json; the ids it feeds are
    checked by running the same prompt through the Python mirror."""
    import subprocess
    from tests.test_tokenizer import _write_tokenizer
    from oracle import tokenizer_oracle as tok_orc
    path = str(tmp_path / "tokenizer.json")
    _write_tokenizer(path)
    exe = os.path.join(os.path.dirname(gpu.capi.LIB_PATH), "llama3_main")
    p = subprocess.run([exe, "--config", "tiny", "--max-pos", "256", "--tokenizer", path, "--text", "hi there",
                        "--decode", "12", "--seed", "5"], capture_output=True, timeout=120)
    assert p.returncode == 0, p.stdout + p.stderr
    enc, dec = tok_orc.load_vocab(path)
    prompt = (b"<|begin_of_text|><|start_header_id|>system<|end_header_id|>\n\nAs a helpful assistant, answer the user "
              b"questions in detail and accurately\n<|eot_id|><|start_header_id|>user<|end_header_id|>\n\nhi there"
              b"\n<|eot_id|><|start_header_id|>assistant<|end_header_id|>\n\n")
    ids = tok_orc.tokenize(enc, prompt)
    cfg = gpu.engine.config("tiny", max_pos=256)
    model = gpu.engine.Model.seeded(cfg, 5).to_device()
    eng = gpu.engine.Engine(model, cfg)
    toks, _ = eng.generate(np.array(ids, np.int32), 12)
    want = b"".join(dec.get(int(t), b"") for t in toks)
    out = p.stdout.split(b"parameters converted to FP16\n", 1)[1]
    assert out == want + b"\n", (out, want)
    eng.close()
    model.close()


@pytest.mark.parametrize("use_graph", [False, True])
@pytest.mark.parametrize("lens", [[5], [7, 40, 3, 21], [500, 20, 515, 9, 64, 130, 2, 33, 77, 5, 6, 90, 100, 250, 11, 12]])
def test_batched_decode_matches_independent_sequences(gpu, lens, use_graph):
    """llama3_decode_batch: sequences of different lengths (one crossing 512 cached positions, which switches
    the whole launch to the span + merge attention) advance together; each must follow its own oracle.  With
    graphs the first step of a (batch size, attention form) runs as plain launches and every later one replays
    one capture, whose kernels read the caches and positions from device memory."""
    cfg = gpu.engine.config("tiny", max_pos=1024)
    model = gpu.engine.Model.seeded(cfg, 17)
    w = H.oracle_weights(model)
    model.to_device()
    B = len(lens)
    engines = [gpu.engine.Engine(model, cfg, use_graph=use_graph) for _ in range(B)]
    oracles = [orc.Model(H.cfg_dict(cfg), w, orc.ORC_REF16) for _ in range(B)]
    cur = []
    for b, n in enumerate(lens):
        prompt = gpu.engine.seeded_tokens(100 + b, n, cfg.vocab)
        t_g, _ = engines[b].prefill(prompt)
        t_o, _, _ = oracles[b].forward(prompt)
        assert t_g == t_o
        cur.append(t_o)
    worst = 0.0
    for step in range(14):
        nxt = gpu.engine.Engine.decode_batch(engines, cur)
        new = []
        for b in range(B):
            t_o, _, lg_o = oracles[b].forward([cur[b]])
            lg_g = engines[0].batch_logits(b)
            e = H.mixed_err(lg_g, lg_o)
            worst = max(worst, e)
            assert H.same_pick_or_near_tie(lg_g, lg_o, nxt[b], t_o), (step, b, nxt[b], t_o)
            new.append(t_o)
        cur = new
        assert [e.pos for e in engines] == [n + step + 1 for n in lens]
    say("batched decode", B, "worst logits err", worst)
    assert worst <= H.TOL
    # a sequence can go on alone afterwards: the single-sequence step sees the rows the batch appended
    t_g, _ = engines[-1].decode(cur[-1])
    t_o, _, _ = oracles[-1].forward([cur[-1]])
    assert t_g == t_o
    for e in engines:
        e.close()
    for o in oracles:
        o.close()
    model.close()


def test_batched_decode_graph_replays_equal_plain_launches(gpu):
    """The captured batched step against plain launches at the 8B layer shapes (2 layers): the same ids and the
    same logits bit for bit on every step, with the set of caches changing between replays (the captured kernels
    read cache pointers and positions from device memory) and a single-sequence step of one member in between."""
    cfg = gpu.engine.config("8b", n_layers=2, max_pos=640)
    model = gpu.engine.Model.seeded(cfg, 23).to_device()
    lens = [30, 7, 500, 64]
    runs = {}
    for use_graph in (False, True):
        engines = [gpu.engine.Engine(model, cfg, use_graph=use_graph) for _ in lens]
        cur = [engines[b].prefill(gpu.engine.seeded_tokens(300 + b, n, cfg.vocab))[0] for b, n in enumerate(lens)]
        trace = []
        for step in range(16):                      # sequence 2 crosses position 512 at step 12: the long form takes over
            order = list(range(4)) if step % 3 else [0, 3, 2, 1]   # caches[0] stays, the others change places
            nxt = gpu.engine.Engine.decode_batch([engines[i] for i in order], [cur[i] for i in order])
            for slot, i in enumerate(order):
                cur[i] = nxt[slot]
                trace.append((step, i, nxt[slot], engines[0].batch_logits(slot).copy()))
            if step == 5:                           # eager work of another kind between two replays
                cur[1] = engines[1].decode(cur[1])[0]
                trace.append((step, 1, cur[1], engines[1].logits()))
        runs[use_graph] = trace
        for e in engines:
            e.close()
    assert len(runs[False]) == len(runs[True])
    for a, b in zip(runs[False], runs[True]):
        assert a[:3] == b[:3] and np.array_equal(a[3], b[3]), a[:3]
    model.close()


def test_sequence_limits(gpu):
    """The cache can be filled to its last row (same ids as the oracle up to there); one row more, an id
    outside the vocabulary or an empty call print the message and exit(1) as the reference's checks do."""
    import subprocess
    import sys
    cfg = gpu.engine.config("tiny", max_pos=64)
    model = gpu.engine.Model.seeded(cfg, 9)
    w = H.oracle_weights(model)
    model.to_device()
    prompt = gpu.engine.seeded_tokens(9, 40, cfg.vocab)
    eng = gpu.engine.Engine(model, cfg)
    toks, _ = eng.generate(prompt, 25)      # rows 0..63 written: the cache is full
    assert eng.pos == 64
    o = orc.Model(H.cfg_dict(cfg), w, orc.ORC_REF16)
    assert [int(t) for t in toks] == o.generate(prompt, 25)
    o.close()
    eng.close()
    model.close()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    head = ("import numpy as np, __graft_entry__ as g\npkg = g.load_package(); pkg.init(0)\n"
            "cfg = pkg.engine.config('tiny', max_pos=64)\nm = pkg.engine.Model.seeded(cfg, 9).to_device()\n"
            "e = pkg.engine.Engine(m, cfg)\np = pkg.engine.seeded_tokens(9, 40, cfg.vocab)\n")
    for body, msg in (("e.generate(p, 25); e.decode(1)", "exceeds max_pos 64"),
                      ("e.generate(p, 26)", "exceed max_pos 64"),
                      ("e.prefill(np.arange(65, dtype=np.int32))", "exceeds max_pos 64"),
                      ("e.prefill(np.array([5, 4096], np.int32))", "outside the vocabulary"),
                      ("e.decode(-1)", "outside the vocabulary"),
                      ("e.inference([])", "empty token list")):
        r = subprocess.run([sys.executable, "-c", head + body], cwd=root, capture_output=True, text=True, timeout=120)
        assert r.returncode == 1 and msg in r.stdout, (body, r.returncode, r.stdout[-300:], r.stderr[-300:])


def test_chunked_prompt_matches_single_pass(gpu):
    cfg, model, eng = _tiny_engine(gpu)
    prompt = gpu.engine.seeded_tokens(8, 50, cfg.vocab)
    t_full, h_full = eng.prefill(prompt, want_hidden=True)
    lg_full = eng.logits()
    eng.reset()
    eng.prefill(prompt[:17])
    eng.prefill(prompt[17:18])  # a one-row chunk goes through the decode kernels
    t_part, h_part = eng.prefill(prompt[18:], want_hidden=True)
    assert t_full == t_part
    assert H.mixed_err(h_part, h_full[:, 18:, :]) <= H.TOL and H.mixed_err(eng.logits(), lg_full) <= H.TOL
    eng.close()
    model.close()


def test_errors_are_reported_not_swallowed(gpu):
    L = gpu.lib()
    assert L.llm_linear(None, 64, None, None, 0, None, 64, 1, 64, 64, None) == gpu.capi.LLM_ERR_INVALID
    assert b"null" in L.llm_last_error()
    buf = gpu.capi.DevBuf((64,), np.uint16)
    assert L.llm_linear(buf.ptr, 60, buf.ptr, None, 0, buf.ptr, 64, 1, 64, 60, None) == gpu.capi.LLM_ERR_INVALID
    # the launches that hand a vector over inside one kernel: a buffer cannot be its own successor, the
    # position must exist, unsupported shapes say so (nothing is launched in any of these calls)
    big = gpu.capi.DevBuf((1 << 16,), np.uint16)
    p = big.ptr
    for fn, extra in ((L.llm_attn_decode_rope_oproj, ()), (L.llm_attn_decode_rope_long_oproj, (p,))):
        args = lambda out, nxt, pos, hq: (p, p, p, out, nxt, pos, None, p, hq, 2, 32, 64) + extra + (p, None, p, 64, p, -1, None)
        assert fn(*args(p, p, 3, 8)) == gpu.capi.LLM_ERR_INVALID and b"refill" in L.llm_last_error()
        assert fn(*args(p, p + 4096, 64, 8)) == gpu.capi.LLM_ERR_INVALID and b"position" in L.llm_last_error()
        assert fn(*args(p, p + 4096, 3, 6)) == gpu.capi.LLM_ERR_INVALID and b"not built" in L.llm_last_error()
    assert L.llm_attn_long_oproj_supported(32, 8, 128, 4096) == 1 and L.llm_attn_long_oproj_supported(32, 8, 128, 1 << 20) == 0
    assert L.llm_attn_long_oproj_supported(6, 2, 32, 64) == 0 and L.llm_attn_oproj_supported(6, 2, 32, 64) == 0


def test_llama3_8b_two_layers_parity(gpu):
    """LLaMA3-8B layer shapes (d 4096, 32/8 heads, FFN 14336, vocab 128256) with 2 layers so the
    oracle finishes in seconds: prompt 24, 8 decode steps.  With random weights the top two of 128256
    logits are often closer than the 2e-2 tolerance, so greedy ids are compared on identical context
    with the near-tie rule of _check_forced, not by demanding equal free-running sequences."""
    cfg = gpu.engine.config("8b", n_layers=2, max_pos=64)
    r = H.run_forced_parity(gpu, cfg, seed=77, n_prompt=24, n_decode=8)
    say({k: v for k, v in r.items() if k not in ("tokens_gpu_free",)})
    _check_forced(r)
    assert max(r["free_hidden_err"]) <= H.TOL and r["free_logits_err"] <= H.TOL
    assert sum(a == b for a, b in zip(r["tokens_oracle"], r["tokens_gpu_forced"])) >= 7


def test_llama3_8b_shapes_at_8k_context(gpu):
    """8192-token prompt in one pass, then decode steps at positions 8192.. (the long-context attention
    kernels, the large GEMM tiles and the KV cache at its real size), 8B layer shapes with 2 layers so that
    the oracle's O(T^2) attention finishes in about a minute."""
    cfg = gpu.engine.config("8b", n_layers=2, max_pos=8256)
    model = gpu.engine.Model.seeded(cfg, 88)
    w = H.oracle_weights(model)
    model.to_device()
    prompt = gpu.engine.seeded_tokens(88, 8192, cfg.vocab)
    eng = gpu.engine.Engine(model, cfg, use_graph=False)
    say("8K context: GPU prompt pass ...")
    tok_g, hid_g = eng.prefill(prompt, want_hidden=True)
    lg_g = eng.logits()
    say("8K context: oracle prompt pass ...")
    o = orc.Model(H.cfg_dict(cfg), w, orc.ORC_REF16)
    tok_o, hid_o, lg_o = o.forward(prompt, want_hidden=True)
    rows = np.r_[0:64, 4064:4128, 8128:8192]
    e_h = [H.mixed_err(hid_g[l][rows], hid_o[l][rows]) for l in range(cfg.n_layers)]
    e_all = H.mixed_err(hid_g, hid_o)
    e_l = H.mixed_err(lg_g, lg_o)
    say("8K context: hidden err", e_h, "all rows", e_all, "logits err", e_l, "tokens", tok_g, tok_o)
    assert e_all <= H.TOL and e_l <= H.TOL
    assert H.same_pick_or_near_tie(lg_g, lg_o, tok_g, tok_o)
    # decode at ctx 8192.. on the oracle's ids
    t = tok_o
    for step in range(6):
        t_g, h_g = eng.decode(int(t), want_hidden=True)
        t_o, h_o, lg_o = o.forward([int(t)], want_hidden=True)
        e = max(H.mixed_err(h_g, h_o), H.mixed_err(eng.logits(), lg_o))
        say("  step", step, "err", e, t_g, t_o)
        assert e <= H.TOL
        assert H.same_pick_or_near_tie(eng.logits(), lg_o, t_g, t_o)
        t = t_o
    o.close()
    eng.close()
    model.close()


def _check_forced(r):
    tol = H.TOL
    assert r["convert_exact"]
    # every layer on identical input: inside the stated tolerance
    assert max(r["forced_hidden_err"]) <= tol, r["forced_hidden_err"]
    assert max(r["forced_decode_hidden_err"]) <= tol, r["forced_decode_hidden_err"]
    assert max(r["forced_logits_err"]) <= tol, r["forced_logits_err"]
    # greedy ids on identical context: equal, or the oracle holds the two ids closer together than
    # the engine's measured logit error at exactly those two ids (no constant allowance)
    for s, (a, b, gap, err) in enumerate(zip(r["tokens_oracle"], r["tokens_gpu_forced"],
                                             r["forced_gap_at_pick"], r["forced_pick_err"])):
        assert a == b or gap <= err, (s, a, b, gap, err)
    # free running, anchored on exact arithmetic: per layer the engine is as close to ORC_FP32 (no
    # intermediate rounding) as the reference's own rounding schedule (ORC_REF16) is.  Both the worst
    # element and the root mean square over the layer; the additive term is one fp16 ulp of the
    # tolerance scale so that layers whose error is a single flipped ulp do not decide the ratio.
    for l in range(len(r["exact_err_hip"])):
        assert r["exact_err_hip"][l] <= 1.5 * r["exact_err_ref16"][l] + 1e-3, (l, r["exact_err_hip"][l], r["exact_err_ref16"][l])
        assert r["exact_rms_hip"][l] <= 1.5 * r["exact_rms_ref16"][l] + 1e-4, (l, r["exact_rms_hip"][l], r["exact_rms_ref16"][l])
    assert r["exact_logits_err_hip"] <= 1.5 * r["exact_logits_err_ref16"] + 1e-3
    # where the free-running ids part from the oracle's (if they do), the oracle's own logits of the
    # two ids differ by less than the model tolerance of the logits
    assert r["free_divergence_gap"] <= 2 * tol * (1 + r.get("free_divergence_logit_scale", 0.0)), r["free_divergence_gap"]
    # ... and by the engine's own logits at that step (same context) the two picks are the same id or a near-tie
    assert r["free_divergence_near_tie"], r
    assert r.get("free_divergence_same_pick_stepwise", True)


def test_llama3_8b_full_depth_parity(gpu):
    """All 32 layers of LLaMA3-8B on seeded weights (about 16 GB on each side), prompt of 128 ids, 32
    greedy steps, against the ORC_REF16 oracle.  Random-init LLaMA at this depth amplifies one-ulp fp16
    rounding differences from layer to layer, so the comparison is made three ways (see
    helpers.run_forced_parity): layer by layer on identical inputs (asserted to 2e-2), free running
    (the engine's distance from unrounded arithmetic, ORC_FP32, asserted to be no more than 1.5x that of
    the reference's own rounding schedule), and on the greedy ids."""
    cfg = gpu.engine.config("8b", max_pos=192)
    say("8B full depth: generating weights, oracle forward ...")
    r = H.run_forced_parity(gpu, cfg, seed=2024, n_prompt=128, n_decode=32)
    say({k: (np.round(v, 4).tolist() if isinstance(v, list) and v and isinstance(v[0], float) else v)
         for k, v in r.items()})
    say("8B full depth: free-running greedy ids identical to the oracle's for the first",
        r["free_identical_prefix"], "of 32; oracle logit gap where they part:", r["free_divergence_gap"])
    _check_forced(r)


def test_tiny_forced_parity(gpu):
    cfg = gpu.engine.config("tiny", max_pos=128)
    r = H.run_forced_parity(gpu, cfg, seed=11, n_prompt=24, n_decode=32)
    _check_forced(r)
    assert r["tokens_gpu_forced"] == r["tokens_oracle"] and r["tokens_gpu_free"] == r["tokens_oracle"]
