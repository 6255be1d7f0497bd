"""CPU tests of the host layer: the C-ABI library loads and exports every
declared symbol, the seeded checkpoint generator matches an independent numpy
restatement, the safetensors loader follows the reference's rules, and the
print-and-exit error behaviour is kept.  No kernel is launched here."""
import ctypes as C
import json
import os
import re
import struct
import subprocess
import sys

import numpy as np
import pytest
from scipy.special import ndtri

from tests import helpers as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- ABI ----------------------------------------------------------------------------
def _declared(header):
    txt = open(os.path.join(ROOT, "include", header)).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    txt = re.sub(r"typedef[^;{}]*\(\s*\*[^;]*;", "", txt)  # function-pointer typedefs
    names = re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{}]*\)\s*;", txt)
    return sorted(set(n for n in names if not n.startswith("llama3_error_fn")))


def test_library_exports_every_declared_symbol(pkg):
    L = pkg.lib()
    for header, table in (("llmcu_hip.h", pkg.capi.HIP_ABI), ("llama3_host.h", pkg.capi.HOST_ABI)):
        declared = [n for n in _declared(header) if n != "llama3_error_fn"]
        assert declared, header
        for name in declared:
            assert hasattr(L, name), "%s declares %s but the library does not export it" % (header, name)
            assert name in table, "%s is declared in %s but has no ctypes binding" % (name, header)
        for name in table:
            assert name in declared, "%s is bound but not declared in %s" % (name, header)


def test_struct_layout_matches_reference_field_order(pkg):
    capi = pkg.capi
    assert [f for f, _ in capi.Tensor._fields_] == ["ndim", "mem_len", "shape", "bf16_tensor", "d_ndim", "d_mem_len",
                                                    "d_shape", "d_bf16_tensor", "d_fp16_tensor"]
    assert [f for f, _ in capi.Llama3Layer._fields_][:2] == ["layernum", "input_layernorm"]
    assert [f for f, _ in capi.Llama3._fields_][:5] == ["embed_tokens", "lm_head", "norm", "layers", "n_layers"]
    assert [f for f, _ in capi.CudaCache._fields_][:9] == ["PN_X", "Q", "K", "V", "d_attention_score_cache",
                                                           "d_feedforward_cache_upgate", "d_token_probdist",
                                                           "h_token_probdist", "f_token_probdist"]


def test_configs(pkg):
    c = pkg.engine.config("8b")
    assert (c.n_layers, c.d_model, c.n_heads, c.n_kv_heads, c.head_dim, c.ffn_dim, c.vocab) == \
        (32, 4096, 32, 8, 128, 14336, 128256)
    assert c.rms_eps == 1e-5 and c.rope_theta == 500000.0 and c.max_pos == 2048
    t = pkg.engine.config("tiny")
    assert (t.n_layers, t.d_model, t.n_heads, t.n_kv_heads, t.head_dim, t.ffn_dim, t.vocab) == \
        (2, 256, 8, 2, 32, 768, 4096)


# ---- seeded generator vs an independent numpy restatement ---------------------------------
M64 = (1 << 64) - 1


def _mix64(z):
    z = (z + 0x9E3779B97F4A7C15) & M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    return z ^ (z >> 31)


def _np_mix64(z):
    z = z + np.uint64(0x9E3779B97F4A7C15)
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def _table(sigma):
    q = ndtri((np.arange(65536) + 0.5) / 65536.0)
    return H.f32_to_bf16((np.float64(np.float32(sigma)) * q).astype(np.float32))


def test_seeded_table_matches_scipy_quantiles(pkg):
    tab = np.ctypeslib.as_array(pkg.lib().seeded_unit_table_bf16(0.02), shape=(65536,))
    want = _table(0.02)
    assert np.array_equal(tab, want)
    v = H.bf16_to_f32(tab).astype(np.float64)
    assert abs(v.mean()) < 1e-6 and abs(v.std() - 0.02) < 2e-4  # N(0, 0.02)


def test_seeded_normal_matches_numpy_restatement(pkg):
    seed, tid, n = 1234, 16 + 16 * 3 + 7, 1003
    got = pkg.engine.seeded_normal_bf16(seed, tid, n)
    key = _mix64(_mix64(seed) ^ tid)
    g = np.arange((n + 3) // 4, dtype=np.uint64)
    with np.errstate(over="ignore"):
        h = _np_mix64(np.uint64(key) + g * np.uint64(0x9E3779B97F4A7C15))
    idx = np.stack([(h >> np.uint64(16 * j)) & np.uint64(0xffff) for j in range(4)], axis=1).reshape(-1)[:n]
    assert np.array_equal(got, _table(0.02)[idx.astype(np.int64)])
    # prefix property: value depends on (seed, id, index) only
    assert np.array_equal(pkg.engine.seeded_normal_bf16(seed, tid, 10), got[:10])
    assert not np.array_equal(pkg.engine.seeded_normal_bf16(seed + 1, tid, n), got)


def test_seeded_tokens_in_range_and_reproducible(pkg):
    t = pkg.engine.seeded_tokens(7, 1000, 4096)
    assert t.min() >= 0 and t.max() < 4096 and len(set(t.tolist())) > 800
    key = _mix64(_mix64(7) ^ 0x746f6b656e73)
    want = [(((_mix64((key + i * 0x9E3779B97F4A7C15) & M64)) >> 32) * 4096) >> 32 for i in range(5)]
    assert t[:5].tolist() == want


# ---- safetensors ---------------------------------------------------------------------------------
def _write_safetensors(path, entries, metadata=True, pad=True):
    """entries: list of (name, dtype, shape, uint16 array)."""
    hdr, off, blobs = {}, 0, []
    if metadata:
        hdr["__metadata__"] = {"format": "pt"}
    for name, dtype, shape, arr in entries:
        b = np.ascontiguousarray(arr).tobytes()
        hdr[name] = {"dtype": dtype, "shape": list(shape), "data_offsets": [off, off + len(b)]}
        off += len(b)
        blobs.append(b)
    js = json.dumps(hdr, separators=(",", ":")).encode()
    if pad:
        js += b" " * ((8 - len(js) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(js)))
        f.write(js)
        for b in blobs:
            f.write(b)


def _tiny_entries(cfg, rng):
    d, qd, kvd, F = cfg.d_model, cfg.n_heads * cfg.head_dim, cfg.n_kv_heads * cfg.head_dim, cfg.ffn_dim
    r = lambda *s: rng.integers(0, 65536, size=s, dtype=np.uint32).astype(np.uint16)
    e = [("model.embed_tokens.weight", "BF16", (cfg.vocab, d), r(cfg.vocab, d)),
         ("lm_head.weight", "BF16", (cfg.vocab, d), r(cfg.vocab, d)),
         ("model.norm.weight", "BF16", (d,), r(d))]
    for l in range(cfg.n_layers):
        p = "model.layers.%d." % l
        e += [(p + "input_layernorm.weight", "BF16", (d,), r(d)),
              (p + "post_attention_layernorm.weight", "BF16", (d,), r(d)),
              (p + "self_attn.q_proj.weight", "BF16", (qd, d), r(qd, d)),
              (p + "self_attn.k_proj.weight", "BF16", (kvd, d), r(kvd, d)),
              (p + "self_attn.v_proj.weight", "BF16", (kvd, d), r(kvd, d)),
              (p + "self_attn.o_proj.weight", "BF16", (d, qd), r(d, qd)),
              (p + "mlp.gate_proj.weight", "BF16", (F, d), r(F, d)),
              (p + "mlp.up_proj.weight", "BF16", (F, d), r(F, d)),
              (p + "mlp.down_proj.weight", "BF16", (d, F), r(d, F))]
    return e


SLOT_OF = {"input_layernorm": "input_layernorm", "post_attention_layernorm": "post_attention_layernorm",
           "q_proj": "self_attn_q_proj", "k_proj": "self_attn_k_proj", "v_proj": "self_attn_v_proj",
           "o_proj": "self_attn_o_proj", "gate_proj": "mlp_gate_proj", "up_proj": "mlp_up_proj",
           "down_proj": "mlp_down_proj"}


def test_loader_places_every_tensor_in_its_slot_across_two_shards(pkg, tmp_path):
    cfg = pkg.engine.config("tiny")
    rng = np.random.default_rng(20)
    entries = _tiny_entries(cfg, rng)
    rng.shuffle(entries)  # file order must not matter
    half = len(entries) // 2
    a, b = str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors")
    _write_safetensors(a, entries[:half])
    _write_safetensors(b, entries[half:], metadata=False, pad=False)
    m = pkg.engine.Model.from_files(cfg, [a, b])
    h = m.host_bf16()
    for name, _, shape, arr in entries:
        if "layers" in name:
            l = int(name.split(".")[2])
            key = [v for k, v in SLOT_OF.items() if "." + k + "." in name or name.split(".")[-2] == k][0]
            got = h[key][l]
        else:
            got = h["embed" if "embed" in name else "lm_head" if "lm_head" in name else "norm"]
        assert got.shape == tuple(shape)
        assert np.array_equal(got, arr), name
    m.close()


def test_loader_reads_file_written_by_the_safetensors_library(pkg, tmp_path):
    torch = pytest.importorskip("torch")
    from safetensors.torch import save_file
    cfg = pkg.engine.config("tiny")
    rng = np.random.default_rng(21)
    entries = _tiny_entries(cfg, rng)
    tensors = {n: torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).reshape(s)
               for n, _, s, a in entries}
    path = str(tmp_path / "lib.safetensors")
    save_file(tensors, path, metadata={"format": "pt"})
    m = pkg.engine.Model.from_files(cfg, [path])
    h = m.host_bf16()
    want = {n: a for n, _, _, a in entries}
    assert np.array_equal(h["embed"], want["model.embed_tokens.weight"])
    assert np.array_equal(h["self_attn_k_proj"][1], want["model.layers.1.self_attn.k_proj.weight"])
    assert np.array_equal(h["mlp_down_proj"][0], want["model.layers.0.mlp.down_proj.weight"])
    m.close()


def test_seeded_safetensors_round_trip_equals_in_memory_fill(pkg, tmp_path):
    cfg = pkg.engine.config("tiny")
    path = str(tmp_path / "seeded.safetensors")
    assert pkg.lib().seeded_write_safetensors(C.byref(cfg), 99, path.encode()) == 0
    a = pkg.engine.Model.from_files(cfg, [path]).host_bf16()
    b = pkg.engine.Model.seeded(cfg, 99).host_bf16()
    for k in a:
        if isinstance(a[k], list):
            for x, y in zip(a[k], b[k]):
                assert np.array_equal(x, y), k
        else:
            assert np.array_equal(a[k], b[k]), k
    assert np.all(b["norm"] == 0x3F80) and np.all(b["input_layernorm"][0] == 0x3F80)  # gains = 1
    # header is valid JSON with HF key names
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        hdr = json.loads(f.read(n))
    assert "model.layers.1.self_attn.q_proj.weight" in hdr and hdr["lm_head.weight"]["dtype"] == "BF16"


# ---- error behaviour: print a message, exit(1) (run in a child process) ----------------------------
def _child(code):
    env = dict(os.environ, PYTHONPATH=ROOT)
    return subprocess.run([sys.executable, "-c", "import __graft_entry__ as ge; pkg = ge.load_package()\n" + code],
                          cwd=ROOT, env=env, capture_output=True, text=True, timeout=120)


def test_missing_file_exits_1_with_the_reference_message():
    p = _child("m = pkg.engine.Model.from_files(pkg.engine.config('tiny'), ['/nonexistent/x.safetensors'])")
    assert p.returncode == 1
    assert "An Error Occurred while opening /nonexistent/x.safetensors" in p.stdout


def test_streaming_loader_reports_missing_files_and_missing_tensors(tmp_path):
    code = ("import ctypes as C\nm = pkg.engine.Model(pkg.engine.config('tiny'))\n"
            "arr = (C.c_char_p * 1)(%r.encode())\npkg.lib().load_safetensor_weights_streaming(m.handle, arr, 1)")
    p = _child(code % "/nonexistent/x.safetensors")
    assert p.returncode == 1 and "An Error Occurred while opening /nonexistent/x.safetensors" in p.stdout
    # a checkpoint that lacks tensors of the model is refused before anything is allocated on a device
    path = str(tmp_path / "partial.safetensors")
    _write_safetensors(path, [("model.norm.weight", "BF16", (256,), np.zeros(256, np.uint16))])
    p = _child(code % path)
    assert p.returncode == 1 and "a tensor was not loaded" in p.stdout


def test_unknown_tensor_name_exits_1(tmp_path):
    path = str(tmp_path / "bad.safetensors")
    _write_safetensors(path, [("model.layers.0.mystery.weight", "BF16", (4,), np.zeros(4, np.uint16))])
    p = _child("pkg.engine.Model.from_files(pkg.engine.config('tiny'), [%r])" % path)
    assert p.returncode == 1 and "Component not allocated" in p.stdout


def test_wrong_dtype_and_bad_layer_and_truncation_exit_1(tmp_path):
    path = str(tmp_path / "f32.safetensors")
    _write_safetensors(path, [("model.norm.weight", "F32", (4,), np.zeros(8, np.uint16))])
    p = _child("pkg.engine.Model.from_files(pkg.engine.config('tiny'), [%r])" % path)
    assert p.returncode == 1 and "not BF16" in p.stdout
    path = str(tmp_path / "layer9.safetensors")
    _write_safetensors(path, [("model.layers.9.mlp.up_proj.weight", "BF16", (4,), np.zeros(4, np.uint16))])
    p = _child("pkg.engine.Model.from_files(pkg.engine.config('tiny'), [%r])" % path)
    assert p.returncode == 1 and "layer 9" in p.stdout
    path = str(tmp_path / "short.safetensors")
    _write_safetensors(path, [("model.norm.weight", "BF16", (64,), np.zeros(8, np.uint16))])
    p = _child("pkg.engine.Model.from_files(pkg.engine.config('tiny'), [%r])" % path)
    assert p.returncode == 1 and "holds 8 of 64" in p.stdout


def test_unparsable_header_prints_and_returns_like_the_reference(tmp_path):
    path = str(tmp_path / "garbage.safetensors")
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", 5) + b"{{{{{")
    p = _child("pkg.engine.Model.from_files(pkg.engine.config('tiny'), [%r]); print('returned')" % path)
    assert p.returncode == 0 and "Error parsing JSON" in p.stdout and "returned" in p.stdout


def test_kernel_entry_points_fail_loudly_without_a_gpu(pkg):
    if pkg.device_count() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(pkg.LlmError):
        pkg.init(0)
