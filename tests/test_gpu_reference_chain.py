"""The reference's own call chain, literally (src/main.cu:61-123 of the reference): init_llama3,
load_safetensor_weights once per shard, to_cuda, init_cache(model) with no configuration, tokens_to_cuda,
then inference() per token on the growing h_tokens array.  A 2-layer checkpoint with the 8B matrix shapes,
seeded, written as two safetensors shards, is driven that way through ctypes and compared with the Engine
path (init_cache_cfg, prefill + decode) and with the CPU oracle; the same two shards then go through
load_safetensor_weights_streaming."""
import ctypes as C
import os

import numpy as np
import pytest

from oracle import pyoracle as orc
from tests import helpers as H
from tests.test_host_layer import _write_safetensors

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def _two_shards(tmp_path, model, cfg):
    """The host tensors of `model` under their Hugging Face names, split over two files the way the real
    checkpoint is: embedding and the first layers in the first, the rest with the final norm and the LM head
    in the second; one layer straddles the boundary."""
    hb = model.host_bf16()
    hf = {"input_layernorm": "input_layernorm.weight", "post_attention_layernorm": "post_attention_layernorm.weight",
          "self_attn_q_proj": "self_attn.q_proj.weight", "self_attn_k_proj": "self_attn.k_proj.weight",
          "self_attn_v_proj": "self_attn.v_proj.weight", "self_attn_o_proj": "self_attn.o_proj.weight",
          "mlp_gate_proj": "mlp.gate_proj.weight", "mlp_up_proj": "mlp.up_proj.weight",
          "mlp_down_proj": "mlp.down_proj.weight"}
    ent = lambda name, a: (name, "BF16", a.shape, a)
    first = [ent("model.embed_tokens.weight", hb["embed"])]
    second = []
    for l in range(cfg.n_layers):
        for i, (slot, name) in enumerate(hf.items()):
            dst = first if (l < cfg.n_layers - 1 or i < 4) else second   # the last layer is split after four tensors
            dst.append(ent("model.layers.%d.%s" % (l, name), hb[slot][l]))
    second += [ent("model.norm.weight", hb["norm"]), ent("lm_head.weight", hb["lm_head"])]
    paths = [str(tmp_path / "model-00001-of-00002.safetensors"), str(tmp_path / "model-00002-of-00002.safetensors")]
    _write_safetensors(paths[0], first)
    _write_safetensors(paths[1], second)
    return paths


def test_reference_call_chain_on_two_shards(gpu, tmp_path):
    lib = gpu.lib()
    cfg = gpu.engine.config("8b", n_layers=2, max_pos=2048)   # what init_cache() derives: head size 128, 2048 positions
    seeded = gpu.engine.Model.seeded(cfg, 77)
    w = H.oracle_weights(seeded)
    paths = _two_shards(tmp_path, seeded, cfg)
    seeded.close()
    n_prompt, n_steps = 12, 8
    prompt = gpu.engine.seeded_tokens(77, n_prompt, cfg.vocab)
    say("shards", [os.path.getsize(p) for p in paths])

    # ---- main.cu:61-93 ------------------------------------------------------------------------------
    model = lib.init_llama3(2)
    for p in paths:
        lib.load_safetensor_weights(model, p.encode())
    lib.to_cuda(model)
    cache = lib.init_cache(model)
    # ---- main.cu:98-123: one chat turn ----------------------------------------------------------------
    h_tokens = np.zeros(2049, np.int32)
    h_tokens[0] = n_prompt + 1
    h_tokens[1:n_prompt + 1] = prompt
    libc = C.CDLL(None)
    libc.malloc.restype, libc.malloc.argtypes = C.c_void_p, [C.c_size_t]
    X = C.cast(libc.malloc(C.sizeof(gpu.capi.Tensor)), C.POINTER(gpu.capi.Tensor))   # main.cu:107: Tensor *X = malloc(...)
    hp = h_tokens.ctypes.data_as(C.POINTER(C.c_int))
    d_tokens = lib.tokens_to_cuda(hp, cfg.d_model, X)
    assert X.contents.shape[0] == 2048 and X.contents.shape[1] == cfg.d_model and X.contents.d_fp16_tensor
    ids, logits = [], []
    for step in range(n_steps):
        nxt = lib.inference(model, X, d_tokens, hp, cache)
        ids.append(int(nxt))
        logits.append(np.ctypeslib.as_array(cache.contents.h_token_probdist, shape=(cfg.vocab,)).copy())
        h_tokens[h_tokens[0]] = nxt          # tokens[tokens[0]] = next_token; tokens[0] += 1 (main.cu:121-122)
        h_tokens[0] += 1
    say("reference chain ids", ids)
    assert lib.llama3_cache_pos(cache) == n_prompt + n_steps - 1
    got_dev = gpu.capi.DevBuf.__new__(gpu.capi.DevBuf)      # the array tokens_to_cuda returned holds what inference() sent up
    got_dev.ptr, got_dev.shape, got_dev.dtype, got_dev.nbytes = C.cast(d_tokens, C.c_void_p).value, (2048,), np.dtype(np.int32), 8192
    up = got_dev.download()
    got_dev.ptr = None
    assert up[0] == h_tokens[0] - 1 and np.array_equal(up[1:n_prompt + n_steps], h_tokens[1:n_prompt + n_steps])

    # ---- the Engine path on a second, separately loaded copy: same bits ---------------------------------
    m2 = gpu.engine.Model.from_files(cfg, paths).to_device()
    eng = gpu.engine.Engine(m2, cfg)
    t, _ = eng.prefill(prompt)
    assert t == ids[0] and np.array_equal(eng.logits(), logits[0])
    for step in range(1, n_steps):
        t, _ = eng.decode(t)
        assert t == ids[step], step
        assert np.array_equal(eng.logits(), logits[step]), step
    eng.close()

    # ---- the oracle ------------------------------------------------------------------------------------
    o = orc.Model(H.cfg_dict(cfg), w, orc.ORC_REF16)
    t_o, _, lg_o = o.forward(prompt)
    worst = 0.0
    for step in range(n_steps):
        err = H.mixed_err(logits[step], lg_o)
        worst = max(worst, err)
        assert err <= H.TOL, (step, err)
        assert ids[step] == t_o, (step, ids[step], t_o)
        if step + 1 < n_steps:
            t_o, _, lg_o = o.forward([t_o])
    o.close()
    say("logits error against the oracle", worst)

    # ---- the same two shards through the streaming loader ------------------------------------------------
    m3 = gpu.engine.Model.from_files_streaming(cfg, paths)
    h2, h3 = m2.handle.contents, m3.handle.contents
    for a, b in ((h2.embed_tokens, h3.embed_tokens), (h2.lm_head, h3.lm_head), (h2.norm, h3.norm)):
        assert np.array_equal(m2.device_fp16(a), m3.device_fp16(b))
    for l in range(cfg.n_layers):
        for slot in gpu.engine.LAYER_SLOTS:
            assert np.array_equal(m2.device_fp16(getattr(h2.layers[l].contents, slot)),
                                  m3.device_fp16(getattr(h3.layers[l].contents, slot))), (l, slot)
    eng3 = gpu.engine.Engine(m3, cfg)
    toks, _ = eng3.generate(prompt, n_steps)
    assert [int(x) for x in toks] == ids
    eng3.close()
    m3.close()
    m2.close()

    lib.free_cache(cache)
    lib._free_tensor(X)   # main.cu:125-126
    gpu.capi.check(lib.llm_free(C.cast(d_tokens, C.c_void_p)))
    lib.free_llama3(model)
    for p in paths:
        os.remove(p)
