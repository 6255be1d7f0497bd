#!/usr/bin/env python3
"""Headline benchmark: LLaMA3-8B batch-1 greedy decode on one MI355X.

A "step" is one decode token through all 32 layers + LM head + argmax with
the KV cache and every weight resident in HBM.  The workload is the full
LLaMA3-8B decoder (32 layers, seeded random-init bf16 weights converted
to fp16 at load, prompt of 128 seeded ids, then K greedy decode steps).  The
same run also measures the 8192-token prompt pass (MFMA GEMM + causal GQA
attention), the dominant kernel (fused gate/up SwiGLU GEMV) against the HBM
roofline with HIP events, and the fp32 CPU port of the reference forward pass
on the host cores as a reported baseline.

    python bench.py [--gpus 1] [--steps 256] [--warmup 8]

Prints ONE JSON line.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12          # B/s, MI355X HBM3E
MFMA_F16_PEAK = 2.5e15     # flop/s, MI355X dense fp16
# HBM bytes one launch of the gate/up SwiGLU GEMV moves, from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) of
# this script, each scaled by the same counter's reading for the calibration copy of kernel_roofline(): kept in a
# small file beside the counter summary, together with the git blob hashes of the kernel sources it was measured
# at.  When a source has changed since, the figure is stale and is not reported.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "decode_gemv_hbm_traffic.json")


def blob_hash(path):
    """git's blob hash of a file (sha1 over 'blob <size>\\0' + content), without needing git."""
    import hashlib
    data = open(path, "rb").read()
    return hashlib.sha1(b"blob %d\0" % len(data) + data).hexdigest()


def measured_traffic():
    """(bytes or None, note) for roofline.traffic."""
    try:
        t = json.load(open(TRAFFIC_FILE))
    except (OSError, ValueError):
        return None, "no counter measurement on file"
    for rel, want in t.get("sources", {}).items():
        if blob_hash(os.path.join(ROOT, rel)) != want:
            return None, "%s changed since the counter run: measure again" % rel
    return int(t["traffic_bytes"]), "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a plain copy (profiles/decode_gemv_hbm_traffic.md)"


def decode_bytes(ctx):
    """Algorithmic HBM bytes of one decode token at context ctx (keys attended):
    every layer's weights + LM head + final norm in fp16, K and V rows of ctx
    positions, one new K/V row, one embedding row."""
    params = 32 * 218112000 + 525336576 + 4096
    return 2 * params + 131072 * ctx + 131072 + 8192


def prefill_flops(T):
    return 2.0 * T * 6979321856 + 262144.0 * T * (T + 1) + 2.0 * 4096 * 128256


def log(*a):
    print("[bench]", *a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--no-prefill-8k", action="store_true")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-steps", type=int, default=8)
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-batch", action="store_true")
    ap.add_argument("--batch-sizes", default="4,16", help="batch sizes of the batched-decode leg (comma separated, 2..16)")
    ap.add_argument("--no-api-loop", action="store_true",
                    help="skip the three inference()-per-token legs (counter runs: thousands of launches less)")
    ap.add_argument("--no-decode-8k", action="store_true", help="skip the 64 decode steps behind the 8192-token prompt")
    ap.add_argument("--ceiling", action="store_true",
                    help="instead of the benchmark: MFMA-only probe and the 8192-token pass with amd-smi power/clock samples")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build measures one MI355X; --gpus %d is not supported "
                 "(no collective path exists, every figure is the one GPU's)" % a.gpus)

    import __graft_entry__ as ge
    pkg = ge.load_package()
    pkg.init(0)
    lib = pkg.lib()
    eng_mod = pkg.engine
    if a.ceiling:
        return power_ceiling(pkg, a)

    cfg = eng_mod.config("8b", max_pos=8704)
    t0 = time.time()
    model = eng_mod.Model.seeded(cfg, a.seed)
    log("seeded bf16 weights on the host in %.1f s" % (time.time() - t0))

    orc = None
    orc_w = None
    if not a.no_cpu_baseline:
        from oracle import pyoracle as orc
        t0 = time.time()
        orc_w = orc.weights_from_bf16(model.host_bf16())  # fp16 copies for the CPU port, before to_cuda frees the bf16
        log("fp16 host copy for the CPU baseline in %.1f s" % (time.time() - t0))

    t0 = time.time()
    model.to_device()
    log("to_cuda (H2D + BF16->FP16 on the device) in %.1f s" % (time.time() - t0))
    engine = eng_mod.Engine(model, cfg, use_graph=not a.no_graph)
    prompt = eng_mod.seeded_tokens(a.seed, a.prompt, cfg.vocab)

    # ---- decode: W untimed warm-up steps, then exactly K timed steps ------------------
    engine.generate(prompt, a.warmup + 1)
    engine.reset()
    pkg.capi.sync()
    w0 = time.time()
    toks, st = engine.generate(prompt, a.steps + 1)   # prompt pass + K decode steps
    pkg.capi.sync()
    wall = time.time() - w0
    K = st.n_decode_steps
    assert K == a.steps
    ms_per_step = st.decode_ms / K
    tok_s = 1e3 / ms_per_step
    ctx_avg = a.prompt + (K + 1) / 2.0  # keys attended, averaged over the timed steps
    frac = decode_bytes(ctx_avg) * tok_s / HBM_PEAK
    log("decode: %d steps in %.2f ms -> %.1f tok/s (%.1f%% of HBM roofline), prompt pass %.2f ms, wall %.2f s"
        % (K, st.decode_ms, tok_s, 100 * frac, st.prefill_ms, wall))

    # ---- the reference's own loop: tokens_to_cuda once, then inference() per token (src/main.cu:109-123) ----
    api = None
    if not a.no_api_loop:
        api = inference_api_loop(pkg, model, engine, cfg, prompt, 64)
        api["sampling_candidates_on_device"] = inference_api_loop(pkg, model, engine, cfg, prompt, 64, "device")
        api["sampling_on_host"] = inference_api_loop(pkg, model, engine, cfg, prompt, 64, "host")
        log("inference() per token, as the reference's main loop drives it: %.1f tok/s (%.3f of llama3_generate)"
            % (api["tok_per_s"], api["tok_per_s"] / tok_s))

    # ---- dominant kernels against their rooflines (HIP events on their own stream) -------------
    roof = kernel_roofline(pkg, model, cfg)
    if not a.no_prefill_8k:
        roof["prefill"] = prefill_kernel_roofline(pkg, model, cfg)

    # ---- 8192-token prompt pass ---------------------------------------------------------------
    prefill = None
    if not a.no_prefill_8k:
        T = 8192
        p8k = eng_mod.seeded_tokens(a.seed + 1, T, cfg.vocab)
        engine.reset()
        engine.generate(p8k, 1)  # warm-up (first use of the large-tile kernels)
        passes = []
        for _ in range(3):  # median of three timed passes
            engine.reset()
            _, st8 = engine.generate(p8k, 1)
            passes.append(st8.prefill_ms)
        ms8 = sorted(passes)[1]
        sec = ms8 * 1e-3
        prefill = {"tokens": T, "ms": ms8, "passes_ms": passes, "tok_per_s": T / sec,
                   "flops": prefill_flops(T), "mfma_frac": prefill_flops(T) / sec / MFMA_F16_PEAK,
                   "peak_tflops": MFMA_F16_PEAK / 1e12}
        log("prefill 8192: %.1f ms -> %.0f tok/s (%.1f%% of fp16 MFMA peak)"
            % (ms8, T / sec, 100 * prefill["mfma_frac"]))
        # long-context decode (KV streaming next to weight streaming), 64 steps at ctx ~8.2K
        if not a.no_decode_8k:
            engine.reset()
            _, stl = engine.generate(p8k, 65)
            ms_l = stl.decode_ms / stl.n_decode_steps
            prefill["decode_at_8k"] = {"steps": stl.n_decode_steps, "ms_per_step": ms_l, "tok_per_s": 1e3 / ms_l,
                                       "hbm_frac": decode_bytes(T + 33) * (1e3 / ms_l) / HBM_PEAK}
            log("decode at ctx 8.2K: %.1f tok/s (%.1f%% of HBM roofline)"
                % (1e3 / ms_l, 100 * prefill["decode_at_8k"]["hbm_frac"]))
    engine.close()

    # ---- batched decode (beyond the reference, which serves one sequence): aggregate tokens/s --------
    batched = None
    if not a.no_batch:
        batched = {}
        bcfg = eng_mod.config("8b", max_pos=512)
        for B in [int(v) for v in a.batch_sizes.split(",") if v]:
            engines = [eng_mod.Engine(model, bcfg, use_graph=not a.no_graph) for _ in range(B)]
            cur = []
            for b, e in enumerate(engines):
                t, _ = e.prefill(eng_mod.seeded_tokens(a.seed + 10 + b, a.prompt, bcfg.vocab))
                cur.append(t)
            for _ in range(4):
                cur = eng_mod.Engine.decode_batch(engines, cur)
            pkg.capi.sync()
            t0 = time.time()
            n_steps = 32
            for _ in range(n_steps):
                cur = eng_mod.Engine.decode_batch(engines, cur)
            pkg.capi.sync()
            dt = time.time() - t0
            batched[str(B)] = {"ms_per_step": 1e3 * dt / n_steps, "tok_per_s": B * n_steps / dt}
            log("batched decode B=%d: %.2f ms per step, %.0f tok/s aggregate" % (B, 1e3 * dt / n_steps, B * n_steps / dt))
            for e in engines:
                e.close()

    # ---- CPU baseline: fp32 port of the reference forward pass on the host cores ---------------
    cpu = None
    if orc is not None:
        cd = {k: getattr(cfg, k) for k, _ in cfg._fields_}
        cd["max_pos"] = 256
        om = orc.Model(cd, orc_w, orc.ORC_FP32)
        t0 = time.time()
        tok, _, _ = om.forward(prompt)
        t_prefill = time.time() - t0
        t0 = time.time()
        for _ in range(a.cpu_steps):
            tok, _, _ = om.forward([tok])
        t_dec = time.time() - t0
        cpu = {"value": a.cpu_steps / t_dec, "unit": "tok/s", "cores": orc.num_threads(), "kind": "port",
               "sample": "%d decode steps after a %d-token prompt on the same seeded LLaMA3-8B weights "
                         "(fp32 activations and accumulation, fp16 weight values)" % (a.cpu_steps, a.prompt),
               "prefill_tok_per_s": a.prompt / t_prefill}
        log("cpu baseline: decode %.2f tok/s, prompt %.1f tok/s on %d threads"
            % (cpu["value"], cpu["prefill_tok_per_s"], cpu["cores"]))
        om.close()
    model.close()

    out = {
        "metric": "LLaMA3-8B bs1 decode tok/s (% HBM roofline); prefill tok/s at 8K (% MFMA)",
        "value": tok_s, "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": a.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16", "data": "synthetic",
        "config": {"workload": "LLaMA3-8B (32 layers, d 4096, 32/8 heads, FFN 14336, vocab 128256), seeded "
                               "random-init bf16 weights converted to fp16 at load, batch 1, prompt %d, %d greedy "
                               "decode steps, fp16 KV cache" % (a.prompt, K),
                   "prompt_tokens": a.prompt, "decode_steps": K, "graph": not a.no_graph},
        "decode_hbm_frac": frac, "decode_bytes_per_token": decode_bytes(ctx_avg),
        "prompt_pass_ms": st.prefill_ms, "inference_api_tok_per_s": api["tok_per_s"] if api else None, "inference_api": api,
        "roofline": roof, "cpu_baseline": cpu, "prefill_8k": prefill, "batched_decode": batched,
        "first_tokens": [int(t) for t in toks[:8]],
    }
    print(json.dumps(out), flush=True)


class SmiSampler:
    """amd-smi power and shader clocks, polled from a thread while something runs on the GPU."""

    def __init__(self):
        import threading
        self.samples, self._stop = [], threading.Event()
        self._t = threading.Thread(target=self._run, daemon=True)

    def _run(self):
        import subprocess
        while not self._stop.is_set():
            try:
                out = subprocess.run(["amd-smi", "metric", "--power", "--clock", "--json"], capture_output=True, text=True,
                                     timeout=5).stdout
                g = json.loads(out)["gpu_data"][0]
                clk = [v["clk"]["value"] for k, v in g["clock"].items() if k.startswith("gfx_") and isinstance(v["clk"], dict)]
                self.samples.append((time.time(), float(g["power"]["socket_power"]["value"]), sum(clk) / max(len(clk), 1)))
            except Exception as e:  # the tool is optional: no samples, no figure
                self.samples.append((time.time(), float("nan"), float("nan")))
                time.sleep(0.2)

    def __enter__(self):
        self._t.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._t.join()

    def window(self, t0, t1):
        w = [(p, c) for t, p, c in self.samples if t0 + 0.15 <= t <= t1 and p == p]
        if not w:
            return {"samples": 0}
        return {"samples": len(w), "power_w_mean": sum(p for p, _ in w) / len(w), "power_w_max": max(p for p, _ in w),
                "gfx_clk_mhz_mean": sum(c for _, c in w) / len(w), "gfx_clk_mhz_min": min(c for _, c in w)}


def power_ceiling(pkg, a):
    """What the board's power limit leaves of the 2.5 PFLOP/s fp16 figure: nothing but MFMAs with constant and with
    random operands, then the 8192-token prompt pass and its gate/up GEMM, each for a second or more with amd-smi
    sampled alongside.  Prints one JSON object."""
    lib, eng_mod = pkg.lib(), pkg.engine
    probe_path = os.path.join(os.path.dirname(pkg.capi.LIB_PATH), "libllmcu_probe.so")
    if not os.path.exists(probe_path):
        raise RuntimeError("%s is missing: run `python llm.cu_amd/build.py`" % probe_path)
    probe = C.CDLL(probe_path)
    probe.mfma_probe.restype = C.c_int
    probe.mfma_probe.argtypes = [C.c_int, C.c_float, C.POINTER(C.c_double), C.POINTER(C.c_float)]
    res = {}
    with SmiSampler() as smi:
        time.sleep(1.0)
        res["idle"] = smi.window(time.time() - 1.0, time.time())
        for kind, name in ((0, "mfma_only_constant_operands"), (1, "mfma_only_random_operands"),
                           (2, "mfma_16x16x32_only_constant_operands"), (3, "mfma_16x16x32_only_random_operands")):
            tf, ms = C.c_double(0), C.c_float(0)
            t0 = time.time()
            rc = probe.mfma_probe(kind, C.c_float(2500.0), C.byref(tf), C.byref(ms))
            if rc != 0:
                raise RuntimeError("mfma_probe(kind %d) failed with code %d" % (kind, rc))
            res[name] = dict(tflops=tf.value, frac_of_2500=tf.value / 2500.0, ms=ms.value, **smi.window(t0, time.time()))
            log(name, res[name])
            time.sleep(1.0)
        cfg = eng_mod.config("8b", max_pos=8192)
        model = eng_mod.Model.seeded(cfg, a.seed).to_device()
        engine = eng_mod.Engine(model, cfg)
        p8k = eng_mod.seeded_tokens(a.seed + 1, 8192, cfg.vocab)
        engine.generate(p8k, 1)
        time.sleep(1.0)
        t0 = time.time()
        passes = []
        for _ in range(12):
            engine.reset()
            _, st8 = engine.generate(p8k, 1)
            passes.append(st8.prefill_ms)
        ms8 = sorted(passes)[len(passes) // 2]
        res["prefill_8192"] = dict(ms=ms8, tflops=prefill_flops(8192) / (ms8 * 1e-3) / 1e12,
                                   frac_of_2500=prefill_flops(8192) / (ms8 * 1e-3) / MFMA_F16_PEAK, **smi.window(t0, time.time()))
        log("prefill_8192", res["prefill_8192"])
        time.sleep(1.0)
        # the gate/up GEMM alone, back to back for about two seconds
        d, F, T = cfg.d_model, cfg.ffn_dim, 8192
        x = pkg.capi.DevBuf.from_host(np.random.default_rng(1).standard_normal((T, d)).astype(np.float16).view(np.uint16))
        hb = pkg.capi.DevBuf((T, F), np.uint16)
        hm = model.handle.contents
        wg = [hm.layers[l].contents.mlp_gate_proj.contents.d_fp16_tensor for l in range(cfg.n_layers)]
        wu = [hm.layers[l].contents.mlp_up_proj.contents.d_fp16_tensor for l in range(cfg.n_layers)]
        timer = pkg.ops.Timer()

        def gemm(stream):
            for l in range(cfg.n_layers):
                pkg.capi.check(lib.llm_linear_swiglu(x.ptr, d, wg[l], wu[l], hb.ptr, F, T, F, d, stream))

        t0 = time.time()
        ms_g = timer.time(gemm, iters=36, warmup=2) / cfg.n_layers
        fl = 2.0 * T * 2 * F * d
        res["gate_up_gemm_8192"] = dict(us=ms_g * 1e3, tflops=fl / (ms_g * 1e-3) / 1e12, frac_of_2500=fl / (ms_g * 1e-3) / MFMA_F16_PEAK,
                                        **smi.window(t0, time.time()))
        log("gate_up_gemm_8192", res["gate_up_gemm_8192"])
        engine.close()
        model.close()
    print(json.dumps(res), flush=True)


def kernel_roofline(pkg, model, cfg):
    """Average duration of the fused gate/up SwiGLU GEMV (the kernel that moves
    most bytes per decode token: 2 x 14336 x 4096 fp16 weights per launch),
    timed with HIP events on the stream it runs on, cycling through the 32
    layers' weights so no launch finds its weights in a cache."""
    lib = pkg.lib()
    ops = pkg.ops
    d, F = cfg.d_model, cfg.ffn_dim
    rng = np.random.default_rng(0)
    x = pkg.capi.DevBuf.from_host(np.ascontiguousarray(rng.standard_normal(d).astype(np.float16)).view(np.uint16))
    out = pkg.capi.DevBuf((F,), np.uint16)
    h = model.handle.contents
    wg = [h.layers[l].contents.mlp_gate_proj.contents.d_fp16_tensor for l in range(cfg.n_layers)]
    wu = [h.layers[l].contents.mlp_up_proj.contents.d_fp16_tensor for l in range(cfg.n_layers)]
    gain = [h.layers[l].contents.post_attention_layernorm.contents.d_fp16_tensor for l in range(cfg.n_layers)]
    timer = ops.Timer()

    def issue(stream):  # the launch the decode step uses: RMSNorm folded into the gate/up GEMV
        for l in range(cfg.n_layers):
            pkg.capi.check(lib.llm_norm_linear_swiglu(x.ptr, gain[l], cfg.rms_eps, wg[l], wu[l], out.ptr, F, d, stream))

    ms = timer.time(issue, iters=8, warmup=2) / cfg.n_layers
    # One plain streaming pass of known size (2^26 elements: 128 MiB read, 128 MiB written) as the
    # calibration dispatch for the FETCH_SIZE / WRITE_SIZE counters; it is the last bf16_to_fp16_kernel
    # dispatch of the run.
    n_cal = 1 << 26
    cal_in = pkg.capi.DevBuf((n_cal,), np.uint16)
    cal_out = pkg.capi.DevBuf((n_cal,), np.uint16)
    pkg.capi.check(lib.llm_fill_zero(cal_in.ptr, n_cal * 2, None))
    pkg.capi.check(lib.llm_bf16_to_fp16(cal_in.ptr, cal_out.ptr, n_cal, None))
    pkg.capi.sync()
    cal_in.free()
    cal_out.free()
    alg = 2 * 2 * F * d + 2 * d + 2 * d + 2 * F  # two weight matrices + activation and gains in + result out
    achieved = alg / (ms * 1e-3)
    traffic, note = measured_traffic()
    return {"kernel": "gemv_kernel<1> = llm_norm_linear_swiglu (RMSNorm + gate/up + SiLU*mul, N=14336, K=4096, T=1)",
            "bound": "hbm", "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
            "frac": achieved / HBM_PEAK, "traffic": traffic, "traffic_note": note, "avg_launch_us": ms * 1e3,
            "algorithmic_bytes_per_launch": alg, "launches_timed": 8 * cfg.n_layers}


def prefill_kernel_roofline(pkg, model, cfg, T=8192):
    """The two kernels that carry the 8192-token prompt pass, timed alone with HIP events on their stream: the
    gate/up GEMM with the SwiGLU epilogue (2 * T * 2F * d flop) and the causal GQA attention (4 * hd * Hq *
    T * (T + 1) / 2 flop: only the keys j <= i are counted)."""
    lib, ops = pkg.lib(), pkg.ops
    d, F, Hq, Hkv, hd = cfg.d_model, cfg.ffn_dim, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim
    rng = np.random.default_rng(1)
    x = pkg.capi.DevBuf.from_host(rng.standard_normal((T, d)).astype(np.float16).view(np.uint16))
    hbuf = pkg.capi.DevBuf((T, F), np.uint16)
    hm = model.handle.contents
    wg = [hm.layers[l].contents.mlp_gate_proj.contents.d_fp16_tensor for l in range(cfg.n_layers)]
    wu = [hm.layers[l].contents.mlp_up_proj.contents.d_fp16_tensor for l in range(cfg.n_layers)]
    timer = ops.Timer()
    n_l = min(cfg.n_layers, 8)

    def gemm(stream):
        for l in range(n_l):
            pkg.capi.check(lib.llm_linear_swiglu(x.ptr, d, wg[l], wu[l], hbuf.ptr, F, T, F, d, stream))

    ms_g = timer.time(gemm, iters=3, warmup=1) / n_l
    fl_g = 2.0 * T * 2 * F * d
    qkv = pkg.capi.DevBuf.from_host((0.5 * rng.standard_normal((T, (Hq + 2 * Hkv) * hd))).astype(np.float16).view(np.uint16))
    kc = pkg.capi.DevBuf.from_host((0.5 * rng.standard_normal((Hkv, T, hd))).astype(np.float16).view(np.uint16))
    vc = pkg.capi.DevBuf.from_host((0.5 * rng.standard_normal((Hkv, hd, T))).astype(np.float16).view(np.uint16))
    ao = pkg.capi.DevBuf((T, Hq * hd), np.uint16)

    def attn(stream):
        pkg.capi.check(lib.llm_attn_prefill(qkv.ptr, (Hq + 2 * Hkv) * hd, kc.ptr, vc.ptr, ao.ptr, Hq * hd, T, 0, Hq, Hkv, hd,
                                            T, stream))

    ms_a = timer.time(attn, iters=8, warmup=2)
    fl_a = 4.0 * hd * Hq * T * (T + 1) / 2
    for b in (x, hbuf, qkv, kc, vc, ao):
        b.free()
    return {"kernel": "gemm_dma64_kernel<2> = llm_linear_swiglu (gate/up + SiLU*mul, T=8192, N=2x14336, K=4096)",
            "bound": "mfma", "flops": fl_g, "avg_us": ms_g * 1e3, "achieved": fl_g / (ms_g * 1e-3) / 1e12,
            "peak": MFMA_F16_PEAK / 1e12, "unit": "TFLOP/s", "frac": fl_g / (ms_g * 1e-3) / MFMA_F16_PEAK,
            "attention": {"kernel": "attn_prefill_pipe_kernel<4> = llm_attn_prefill (T=8192, 32/8 heads, causal)",
                          "flops": fl_a, "avg_us": ms_a * 1e3, "achieved": fl_a / (ms_a * 1e-3) / 1e12,
                          "frac": fl_a / (ms_a * 1e-3) / MFMA_F16_PEAK}}


def inference_api_loop(pkg, model, engine, cfg, prompt, n_tokens, sampling=None):
    """The reference's token loop (src/main.cu:109-123) against this library: tokens_to_cuda once, then one
    inference() call per generated token on the growing token array; wall-clock per call from the second call on
    (the first call is the prompt pass).  sampling: None = greedy ids; "device" / "host" = the reference's
    sampler (temperature 0.7, top-k 50, top-p 0.9) with the candidates selected on the device / everything
    on the host."""
    lib = pkg.lib()
    engine.reset()
    engine.set_sampling(sampling is not None)
    engine.set_device_sampling(sampling != "host")
    tokens = np.zeros(2049, np.int32)
    n = len(prompt)
    tokens[0] = n + 1
    tokens[1:n + 1] = prompt
    libc = C.CDLL("libc.so.6")
    libc.malloc.restype = C.c_void_p
    X = C.cast(libc.malloc(C.sizeof(pkg.capi.Tensor)), C.POINTER(pkg.capi.Tensor))  # _free_tensor frees it, as in main.cu
    tp = tokens.ctypes.data_as(C.POINTER(C.c_int))
    d_tokens = lib.tokens_to_cuda(tp, cfg.d_model, X)
    nxt = lib.inference(model.handle, X, d_tokens, tp, engine.cache)  # prompt pass
    out = [int(nxt)]
    tokens[tokens[0]] = nxt
    tokens[0] += 1
    for _ in range(4):  # warm-up decode calls (graph capture)
        nxt = lib.inference(model.handle, X, d_tokens, tp, engine.cache)
        out.append(int(nxt))
        tokens[tokens[0]] = nxt
        tokens[0] += 1
    t0 = time.time()
    for _ in range(n_tokens):
        nxt = lib.inference(model.handle, X, d_tokens, tp, engine.cache)
        tokens[tokens[0]] = nxt
        tokens[0] += 1
    dt = time.time() - t0
    lib._free_tensor(X)
    pkg.capi.check(lib.llm_free(C.cast(d_tokens, C.c_void_p)))
    engine.reset()
    engine.set_sampling(False)
    engine.set_device_sampling(True)
    if sampling is not None:
        return {"tokens": n_tokens, "ms_per_call": 1e3 * dt / n_tokens, "tok_per_s": n_tokens / dt}
    return {"tokens": n_tokens, "ms_per_call": 1e3 * dt / n_tokens, "tok_per_s": n_tokens / dt,
            "what": "tokens_to_cuda once, then inference(model, X, d_tokens, h_tokens, cache) per token; each call returns "
                    "the greedy id and leaves the fp16 logits in cache->h_token_probdist (one stream sync per call)"}


if __name__ == "__main__":
    main()
