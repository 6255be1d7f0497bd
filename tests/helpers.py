"""Shared pieces of the parity tests: numpy float64 closed forms, the mixed
abs/rel error the north star states (2e-2), and the whole-model comparison of
the HIP engine with the CPU oracle on identical seeded weights."""
import numpy as np

from oracle import pyoracle as orc

TOL = 2e-2  # max-abs/rel tolerance for fp16 hidden states and logits


def f16(bits):
    return np.ascontiguousarray(bits).view(np.float16).astype(np.float64)


def bits(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float16)).view(np.uint16)


def mixed_err(a_bits, b_bits):
    """max_i |a-b| / (1 + |b|).  err <= tol is |a-b| <= tol + tol*|b| for every element, i.e.
    numpy.allclose(a, b, atol=tol, rtol=tol): the max-abs / rel tolerance with both set to tol."""
    a, b = f16(a_bits), f16(b_bits)
    return float(np.max(np.abs(a - b) / (1.0 + np.abs(b)))) if a.size else 0.0


def same_pick_or_near_tie(lg_gpu, lg_orc, t_gpu, t_orc):
    """Greedy ids on identical context: equal, or the oracle's own logits of the two ids are no
    further apart than the engine's measured error at exactly those two logits (which the caller
    bounds by the tolerance separately)."""
    if int(t_gpu) == int(t_orc):
        return True
    g, o = f16(lg_gpu), f16(lg_orc)
    return float(o[t_orc] - o[t_gpu]) <= float(abs(g[t_orc] - o[t_orc]) + abs(g[t_gpu] - o[t_gpu]))


def rms_err(a_bits, b_bits):
    """root mean square of a-b over the root mean square of b."""
    a, b = f16(a_bits), f16(b_bits)
    return float(np.sqrt(np.mean((a - b) ** 2) / max(np.mean(b * b), 1e-30)))


def ulp_diff(a_bits, b_bits):
    """distance in fp16 ulps (monotone integer mapping of the bit patterns)."""
    def key(x):
        x = np.ascontiguousarray(x).astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7fff), x & 0x7fff)
    return np.abs(key(a_bits) - key(b_bits))


def bf16_to_f32(b):
    return (np.ascontiguousarray(b).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def cfg_dict(cfg):
    return {k: getattr(cfg, k) for k, _ in cfg._fields_}


def oracle_weights(model):
    """fp16 weights for the oracle from a host-side (not yet uploaded) Model."""
    return orc.weights_from_bf16(model.host_bf16())


def run_model_parity(pkg, cfg, seed, n_prompt, n_decode, use_graph=True, oracle_decode=None):
    """Runs prompt + greedy decode on the HIP engine and on the ORC_REF16
    oracle from the same seeded bf16 weights and prompt.  Returns errors and
    both token sequences.  oracle_decode limits how many decode steps the
    oracle follows (default: all)."""
    eng_mod = pkg.engine
    model = eng_mod.Model.seeded(cfg, seed)
    w = oracle_weights(model)
    model.to_device()
    prompt = eng_mod.seeded_tokens(seed, n_prompt, cfg.vocab)
    out = {}
    # weight conversion must be bit-exact
    dev_embed = model.device_fp16(model.handle.contents.embed_tokens)
    out["convert_exact"] = bool(np.array_equal(dev_embed, w["embed"]))

    engine = eng_mod.Engine(model, cfg, use_graph=use_graph)
    o = orc.Model(cfg_dict(cfg), w, orc.ORC_REF16)

    tok_g, hid_g = engine.prefill(prompt, want_hidden=True)
    logits_g = engine.logits()
    tok_o, hid_o, logits_o = o.forward(prompt, want_hidden=True)
    out["hidden_max_err"] = max(mixed_err(hid_g[l], hid_o[l]) for l in range(cfg.n_layers))
    out["hidden_err_per_layer"] = [mixed_err(hid_g[l], hid_o[l]) for l in range(cfg.n_layers)]
    out["logits_max_err"] = mixed_err(logits_g, logits_o)
    out["argmax_matches_own_logits"] = bool(tok_g == orc.argmax_f16(logits_g))
    out["first_token"] = (int(tok_g), int(tok_o))

    # greedy decode: device-resident loop vs oracle
    engine.reset()
    toks_g, stats = engine.generate(prompt, n_decode)
    n_o = n_decode if oracle_decode is None else min(n_decode, oracle_decode)
    toks_o = [int(tok_o)]
    gaps = []
    for _ in range(n_o - 1):
        t, _, lg = o.forward([toks_o[-1]])
        v = np.sort(f16(lg))
        gaps.append(float(v[-1] - v[-2]))
        toks_o.append(int(t))
    out["tokens_gpu"] = [int(t) for t in toks_g[:n_o]]
    out["tokens_oracle"] = toks_o
    out["top2_gaps"] = gaps
    out["stats"] = {"prefill_ms": stats.prefill_ms, "decode_ms": stats.decode_ms,
                    "n_decode_steps": stats.n_decode_steps}
    out["tokens_all_gpu"] = [int(t) for t in toks_g]
    o.close()
    engine.close()
    model.close()
    return out


def run_forced_parity(pkg, cfg, seed, n_prompt, n_decode):
    """Full-depth comparison that separates kernel error from the compounding of fp16 rounding
    differences across layers:
      forced_*  every layer (and every decode step) of the HIP engine starts from the oracle's own
                previous-layer output, so the error of each layer stands alone;
      free_*    the engine runs on its own, errors compound;
      floor_*   ORC_REF16 against ORC_REF16_REV (the oracle with every projection summed over k in
                the opposite order): what a legal fp32 reordering of the reference's own arithmetic
                does to the same hidden states;
      exact_*   distance of each of the three (ORC_REF16, ORC_REF16_REV, the free-running engine) from
                ORC_FP32, the same graph with no intermediate rounding: how close each rounding
                schedule stays to exact arithmetic."""
    eng_mod = pkg.engine
    model = eng_mod.Model.seeded(cfg, seed)
    w = oracle_weights(model)
    model.to_device()
    prompt = eng_mod.seeded_tokens(seed, n_prompt, cfg.vocab)
    L = cfg.n_layers
    out = {}
    out["convert_exact"] = bool(np.array_equal(model.device_fp16(model.handle.contents.lm_head), w["lm_head"]))
    engine = eng_mod.Engine(model, cfg, use_graph=False)
    o = orc.Model(cfg_dict(cfg), w, orc.ORC_REF16)
    o_rev = orc.Model(cfg_dict(cfg), w, orc.ORC_REF16_REV)
    tok_o, hid_o, lg_o = o.forward(prompt, want_hidden=True)
    _, hid_r, lg_r = o_rev.forward(prompt, want_hidden=True)
    out["floor_hidden_err"] = [mixed_err(hid_r[l], hid_o[l]) for l in range(L)]
    out["floor_logits_err"] = mixed_err(lg_r, lg_o)
    o_rev.close()
    o_x = orc.Model(cfg_dict(cfg), w, orc.ORC_FP32)
    _, hid_x, lg_x = o_x.forward(prompt, want_hidden=True)
    o_x.close()
    out["exact_err_ref16"] = [mixed_err(hid_o[l], hid_x[l]) for l in range(L)]
    out["exact_err_rev"] = [mixed_err(hid_r[l], hid_x[l]) for l in range(L)]
    out["exact_rms_ref16"] = [rms_err(hid_o[l], hid_x[l]) for l in range(L)]
    out["exact_rms_rev"] = [rms_err(hid_r[l], hid_x[l]) for l in range(L)]
    out["exact_logits_err_ref16"] = mixed_err(lg_o, lg_x)
    # free running
    tok_f, hid_f = engine.prefill(prompt, want_hidden=True)
    out["exact_err_hip"] = [mixed_err(hid_f[l], hid_x[l]) for l in range(L)]
    out["exact_rms_hip"] = [rms_err(hid_f[l], hid_x[l]) for l in range(L)]
    out["exact_logits_err_hip"] = mixed_err(engine.logits(), lg_x)
    out["free_hidden_err"] = [mixed_err(hid_f[l], hid_o[l]) for l in range(L)]
    out["free_logits_err"] = mixed_err(engine.logits(), lg_o)
    out["free_first_token"] = (int(tok_f), int(tok_o))
    # teacher forced prompt pass
    engine.reset()
    tok_g, hid_g = engine.prefill(prompt, want_hidden=True, inject=hid_o)
    lg_g = engine.logits()
    out["forced_hidden_err"] = [mixed_err(hid_g[l], hid_o[l]) for l in range(L)]
    out["forced_logits_err"] = [mixed_err(lg_g, lg_o)]
    # teacher forced greedy steps: both sides consume the oracle's tokens
    toks_o, toks_g, gaps, dec_err, pick_err, lg_steps = [int(tok_o)], [int(tok_g)], [], [], [], [lg_o]
    top = f16(lg_o)
    gaps.append(float(top.max() - top[tok_g]))
    pick_err.append(float(abs(f16(lg_g)[tok_o] - top[tok_o]) + abs(f16(lg_g)[tok_g] - top[tok_g])))
    for _ in range(n_decode - 1):
        t_o, h_o, lg_o = o.forward([toks_o[-1]], want_hidden=True)
        t_g, h_g = engine.decode(toks_o[-1], want_hidden=True, inject=h_o)
        lg_g = engine.logits()
        dec_err.append(max(mixed_err(h_g[l], h_o[l]) for l in range(L)))
        out["forced_logits_err"].append(mixed_err(lg_g, lg_o))
        top = f16(lg_o)
        gaps.append(float(top.max() - top[t_g]))  # 0 when both picked the same id
        pick_err.append(float(abs(f16(lg_g)[t_o] - top[t_o]) + abs(f16(lg_g)[t_g] - top[t_g])))
        lg_steps.append(lg_o)
        toks_o.append(int(t_o))
        toks_g.append(int(t_g))
    out["forced_decode_hidden_err"] = dec_err
    out["tokens_oracle"], out["tokens_gpu_forced"], out["forced_gap_at_pick"] = toks_o, toks_g, gaps
    out["forced_pick_err"] = pick_err  # |engine - oracle| logit error summed over the two ids picked
    # free-running greedy tokens (device-resident loop) for the record
    engine.close()
    engine = eng_mod.Engine(model, cfg, use_graph=True)
    free, _ = engine.generate(prompt, n_decode)
    out["tokens_gpu_free"] = [int(t) for t in free]
    same = 0
    for a, b in zip(out["tokens_gpu_free"], toks_o):
        if a != b:
            break
        same += 1
    out["free_identical_prefix"] = same
    # at the first step where the free-running ids part, both sides still had identical context:
    # how far apart the oracle itself holds the two ids there
    if same < len(toks_o):
        top = f16(lg_steps[same])
        out["free_divergence_gap"] = float(top[toks_o[same]] - top[out["tokens_gpu_free"][same]])
        out["free_divergence_logit_scale"] = float(np.abs(top).max())
        # the engine's own logits at that step, on the same context (step by step up to the parting step):
        # the two picks must be a near-tie by the engine's measured error at exactly those two logits
        engine.reset()
        t, _ = engine.prefill(prompt)
        for i in range(same):
            assert int(t) == toks_o[i]
            t, _ = engine.decode(toks_o[i])
        out["free_divergence_same_pick_stepwise"] = bool(int(t) == out["tokens_gpu_free"][same])
        out["free_divergence_near_tie"] = bool(same_pick_or_near_tie(engine.logits(), lg_steps[same], int(t), toks_o[same]))
    else:
        out["free_divergence_gap"] = 0.0
        out["free_divergence_near_tie"] = True
    o.close()
    engine.close()
    model.close()
    return out


# ---- float64 closed forms ------------------------------------------------------
def rmsnorm_f64(x, g, eps=1e-5):
    x, g = f16(x), f16(g)
    rms = np.sqrt(eps + np.mean(x * x, axis=-1, keepdims=True))
    return x * g / rms


def rope_f64(x, n_heads, head_dim, pos0=0, theta=500000.0):
    x = f16(x).reshape(x.shape[0], n_heads, head_dim // 2, 2)
    T = x.shape[0]
    i = np.arange(head_dim // 2, dtype=np.float64)
    freq = theta ** (-2.0 * i / head_dim)
    ang = (pos0 + np.arange(T, dtype=np.float64))[:, None] * freq[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    e, o = x[..., 0], x[..., 1]
    out = np.stack([c * e - s * o, s * e + c * o], axis=-1)
    return out.reshape(T, n_heads * head_dim)


def attention_f64(q, k, v, pos0, n_heads, n_kv_heads, head_dim):
    q, k, v = f16(q), f16(k), f16(v)
    Tq = q.shape[0]
    g = n_heads // n_kv_heads
    out = np.zeros_like(q)
    for h in range(n_heads):
        kv = h // g
        qh = q[:, h * head_dim:(h + 1) * head_dim]
        kh = k[:, kv * head_dim:(kv + 1) * head_dim]
        vh = v[:, kv * head_dim:(kv + 1) * head_dim]
        for t in range(Tq):
            n = pos0 + t + 1
            s = kh[:n] @ qh[t] / np.sqrt(head_dim)
            p = np.exp(s - s.max())
            p /= p.sum()
            out[t, h * head_dim:(h + 1) * head_dim] = p @ vh[:n]
    return out


def silu(x):
    return x / (1.0 + np.exp(-x))


def model_forward_f64(cfg, w, tokens, mutate=None):
    """Independent float64 forward of the whole model, composed from the closed forms above and
    plain `@`, wired as the reference's driver is (src/inference/inference.cu:149-193): embedding;
    per layer  x += Wo.attn(rope(Wq.n), rope(Wk.n), Wv.n) with n = norm(x, input_ln),  then
    x += Wdown.(silu(Wgate.m) * (Wup.m)) with m = norm(x, post_ln);  final norm; LM head on the last
    row only (inference.cu:1014).  No intermediate rounding.  Returns (hidden [L,T,d], logits [V]).
    `mutate` names one deliberate wiring mistake, used to show that the comparison would catch it."""
    d, Hq, Hkv, hd = cfg["d_model"], cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    eps, theta = cfg.get("rms_eps", 1e-5), cfg.get("rope_theta", 500000.0)
    W = lambda a: f16(a)
    norm = lambda x, g: x * W(g) / np.sqrt(eps + np.mean(x * x, axis=-1, keepdims=True))
    T = len(tokens)

    def rope(x, n_heads):
        x = x.reshape(T, n_heads, hd // 2, 2)
        ang = np.arange(T, dtype=np.float64)[:, None] * theta ** (-2.0 * np.arange(hd // 2) / hd)[None, :]
        c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
        return np.stack([c * x[..., 0] - s * x[..., 1], s * x[..., 0] + c * x[..., 1]], -1).reshape(T, n_heads * hd)

    def attention(q, k, v):
        out = np.zeros((T, Hq * hd))
        for h in range(Hq):
            kv = h // (Hq // Hkv)
            s = q[:, h * hd:(h + 1) * hd] @ k[:, kv * hd:(kv + 1) * hd].T / np.sqrt(hd)
            s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
            p = np.exp(s - s.max(axis=1, keepdims=True))
            out[:, h * hd:(h + 1) * hd] = (p / p.sum(axis=1, keepdims=True)) @ v[:, kv * hd:(kv + 1) * hd]
        return out

    x = W(w["embed"])[np.asarray(tokens)]
    hidden = []
    for l in range(cfg["n_layers"]):
        g_in, g_post = w["input_ln"][l], w["post_ln"][l]
        if mutate == "swap_norm_gains":
            g_in, g_post = g_post, g_in
        n = norm(x, g_in)
        q, k, v = n @ W(w["wq"][l]).T, n @ W(w["wk"][l]).T, n @ W(w["wv"][l]).T
        if mutate != "no_rope":
            q, k = rope(q, Hq), rope(k, Hkv)
        a = attention(q, k, v) @ W(w["wo"][l]).T
        x = (n if mutate == "residual_after_norm" else x) + a
        m = norm(x, g_post)
        gate, up = m @ W(w["wgate"][l]).T, m @ W(w["wup"][l]).T
        if mutate == "swap_gate_up":
            gate, up = up, gate
        x = x + (silu(gate) * up) @ W(w["wdown"][l]).T
        hidden.append(x.copy())
    last = x[-1] if mutate == "no_final_norm" else norm(x[-1:], w["norm"])[0]
    return np.stack(hidden), last @ W(w["lm_head"]).T
