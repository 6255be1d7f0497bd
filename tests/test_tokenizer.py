"""Tokenizer of the reference (src/tokenizer/tokenizer.cu): shipped trie tokenizer against the oracle's
restatement on a synthetic Hugging Face tokenizer.json (the real one is not in the reference tree).  CPU only."""
import ctypes as C
import json
import subprocess
import sys
import os

import numpy as np
import pytest

from oracle import tokenizer_oracle as tok_orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DECODE_SIZE = 600


def _write_tokenizer(path):
    """Single bytes for printable ASCII, overlapping multi-byte pieces, UTF-8 pieces, special tokens."""
    vocab = {}
    nid = 0
    for c in range(32, 127):
        vocab[chr(c)] = nid
        nid += 1
    vocab["\n"] = nid; nid += 1
    for piece in ["th", "the", "there", "he", "her", "here", " the", " a", "an", "and", " and", "ing", "in", "at",
                  "ation", "é", "ée", "日", "日本", "日本語", "\n\n", "  ", "    ", "ab", "abc", "abcd", "bcd", "user",
                  "system", "assistant"]:
        vocab[piece] = nid
        nid += 1
    added = [{"id": 500 + i, "content": s} for i, s in enumerate(
        ["<|begin_of_text|>", "<|start_header_id|>", "<|end_header_id|>", "<|eot_id|>"])]
    added.append({"id": 599, "content": "the"})       # an added token that repeats a vocabulary string
    with open(path, "w", encoding="utf-8") as f:
        json.dump({"added_tokens": added, "model": {"type": "BPE", "vocab": vocab}}, f, ensure_ascii=False)
    return vocab, added


def test_oracle_on_hand_worked_examples_and_brute_force(tmp_path):
    path = str(tmp_path / "tokenizer.json")
    vocab, added = _write_tokenizer(path)
    enc, dec = tok_orc.load_vocab(path)
    # "there" beats "the"/"th"; the added "the" (599) replaced the vocabulary id; " the" is its own piece
    assert tok_orc.tokenize(enc, b"there") == [vocab["there"]]
    assert tok_orc.tokenize(enc, b"the") == [599]
    assert tok_orc.tokenize(enc, b"then") == [599, vocab["n"]]
    assert tok_orc.tokenize(enc, b" there") == [vocab[" the"], vocab["r"], vocab["e"]]   # greedy, not optimal
    assert tok_orc.tokenize(enc, b"abcd") == [vocab["abcd"]]
    assert tok_orc.tokenize(enc, b"abce") == [vocab["abc"], vocab["e"]]
    assert tok_orc.tokenize(enc, "日本語日".encode()) == [vocab["日本語"], vocab["日"]]
    assert tok_orc.tokenize(enc, b"<|eot_id|>x") == [503, vocab["x"]]
    with pytest.raises(ValueError) as e:
        tok_orc.tokenize(enc, b"ok\x01")
    assert e.value.args[0] == 2
    # brute force: at every step the chosen piece is the longest vocabulary entry that prefixes the rest,
    # provided every shorter prefix of it is a prefix of some entry (always true here: single bytes exist)
    rng = np.random.default_rng(0)
    alphabet = list("theran dbc\n") + ["é", "日", "日本", "日本語"]
    for _ in range(200):
        text = "".join(rng.choice(alphabet, size=int(rng.integers(1, 40)))).encode()
        ids = tok_orc.tokenize(enc, text)
        i = 0
        for t in ids:
            cands = [k for k in enc if text.startswith(k, i)]
            assert dec[t] == max(cands, key=len)
            i += len(dec[t])
        assert i == len(text) and b"".join(dec[t] for t in ids) == text


def _lib(pkg):
    return pkg.lib()


def test_shipped_tokenizer_equals_oracle_and_decodes_back(pkg, tmp_path):
    lib = _lib(pkg)
    path = str(tmp_path / "tokenizer.json")
    vocab, added = _write_tokenizer(path)
    enc, dec = tok_orc.load_vocab(path)
    tk = lib.load_tokenizer_from(path.encode(), DECODE_SIZE)

    class Tok(C.Structure):
        _fields_ = [("root", C.c_void_p), ("decode", C.POINTER(C.c_char_p))]

    t = C.cast(tk, C.POINTER(Tok)).contents
    for i, b in dec.items():
        assert t.decode[i] == b
    assert t.decode[400] is None          # ids nobody defined stay NULL
    libc = C.CDLL("libc.so.6")
    rng = np.random.default_rng(1)
    alphabet = list("theran dbcing at\n <>|_") + ["é", "日", "日本", "日本語", "<|eot_id|>", "<|begin_of_text|>", "    "]
    texts = [b"there and here", "日本語 ée".encode()]
    texts += ["".join(rng.choice(alphabet, size=int(rng.integers(1, 200)))).encode() for _ in range(300)]
    for text in texts:
        arr = lib.tokenize(tk, text)
        n = arr[0] - 1
        got = [arr[1 + i] for i in range(n)]
        libc.free(arr)
        assert got == tok_orc.tokenize(enc, text)
        assert b"".join(t.decode[i] for i in got) == text
    # the 2048-token cap (tokenizer.cu:119): input beyond it is dropped, tokens[0] = 2049
    long_text = b"x" * 5000
    arr = lib.tokenize(tk, long_text)
    assert arr[0] == 2049 and all(arr[1 + i] == vocab["x"] for i in range(2048))
    libc.free(arr)
    assert tok_orc.tokenize(enc, long_text) == [vocab["x"]] * 2048
    # the chat template of main.cu:26-59 tokenizes into the special ids around the user text
    lib.llama3_chat_prompt.restype = C.c_void_p
    p = lib.llama3_chat_prompt(b"hi there")
    prompt = C.string_at(p)
    libc.free(C.c_void_p(p))
    assert prompt.startswith(b"<|begin_of_text|><|start_header_id|>system<|end_header_id|>\n\nAs a helpful assistant")
    assert prompt.endswith(b"user<|end_header_id|>\n\nhi there\n<|eot_id|><|start_header_id|>assistant<|end_header_id|>\n\n")
    arr = lib.tokenize(tk, prompt)
    got = [arr[1 + i] for i in range(arr[0] - 1)]
    libc.free(arr)
    assert got == tok_orc.tokenize(enc, prompt) and got[0] == 500 and got[1] == 501
    lib.free_tokenizer(tk, DECODE_SIZE)


def _child(code):
    full = "import __graft_entry__ as g, ctypes as C\npkg = g.load_package()\nlib = pkg.lib()\n" + code
    return subprocess.run([sys.executable, "-c", full], cwd=ROOT, capture_output=True, text=True, timeout=120)


def test_failures_print_and_exit_like_the_reference(tmp_path):
    path = str(tmp_path / "tokenizer.json")
    _write_tokenizer(path)
    p = _child("tk = lib.load_tokenizer_from(%r.encode(), 600)\nlib.tokenize(tk, b'ok\\x01')" % path)
    assert p.returncode == 1 and "Error: Unable to tokenize input at position 2" in p.stdout
    p = _child("lib.load_tokenizer_from(b'/nonexistent/tokenizer.json', 600)")
    assert p.returncode == 1 and "Could not determine file size" in p.stdout
    bad = str(tmp_path / "bad.json")
    open(bad, "w").write('{"model": {"vocab": {"a": 0}}}')
    p = _child("lib.load_tokenizer_from(%r.encode(), 600)" % bad)
    assert p.returncode == 1 and "added_tokens" in p.stdout
    open(bad, "w").write('{"added_tokens": [], "model": {"vocab": {"a": 700}}}')
    p = _child("lib.load_tokenizer_from(%r.encode(), 600)" % bad)
    assert p.returncode == 1 and "outside the decode table" in p.stdout
    # the reference's own entry point looks for model_weights/modified_tokenizer.json
    p = _child("lib.load_tokenizer()")
    assert p.returncode == 1 and "Could not determine file size" in p.stdout


class _Node(C.Structure):
    pass


_Node._fields_ = [("_max_childs", C.c_int), ("child_len", C.c_int), ("child_char", C.POINTER(C.c_ubyte)),
                  ("child_node", C.POINTER(C.POINTER(_Node))), ("token", C.c_int)]


def _walk(node, prefix, out):
    """every (string, id) a trie holds; checks the ordering invariant and the capacity on the way"""
    n = node.contents
    assert 0 <= n.child_len <= n._max_childs
    bytes_ = [n.child_char[i] for i in range(n.child_len)]
    assert bytes_ == sorted(set(bytes_)), bytes_          # ascending unsigned bytes, no duplicates
    if n.token != -1:
        out[bytes(prefix)] = n.token
    for i in range(n.child_len):
        _walk(n.child_node[i], prefix + [bytes_[i]], out)


def test_trie_built_at_once_and_string_by_string_hold_the_same_vocabulary(pkg, tmp_path):
    """The loader lays the trie down from the sorted vocabulary in one pass; the exported _build_trie splices
    one string at a time into place.  Both keep a node's children sorted by unsigned byte (what _find_child's
    binary search needs) and both hold exactly the oracle's vocabulary, whatever the insertion order; a trie
    made by hand tokenizes like the loaded one."""
    lib = _lib(pkg)
    path = str(tmp_path / "tokenizer.json")
    _write_tokenizer(path)
    enc, _ = tok_orc.load_vocab(path)
    tk = lib.load_tokenizer_from(path.encode(), DECODE_SIZE)

    class Tok(C.Structure):
        _fields_ = [("root", C.POINTER(_Node)), ("decode", C.c_void_p)]

    loaded = {}
    _walk(C.cast(tk, C.POINTER(Tok)).contents.root, [], loaded)
    assert loaded == enc
    lib.init_trienode.restype = C.POINTER(_Node)
    lib._build_trie.argtypes = [C.POINTER(_Node), C.c_char_p, C.c_int]
    lib._find_child.argtypes = [C.POINTER(_Node), C.c_char, C.POINTER(C.POINTER(_Node))]
    rng = np.random.default_rng(4)
    items = list(enc.items())
    for trial in range(3):
        order = rng.permutation(len(items))
        root = lib.init_trienode()
        lib._build_trie(root, b"the", 12345)              # replaced below: the later definition of a string stays
        for j in order:
            lib._build_trie(root, items[j][0], items[j][1])
        built = {}
        _walk(root, [], built)
        assert built == enc
        hit = C.POINTER(_Node)()
        assert lib._find_child(root, b"t", C.byref(hit)) >= 0 and lib._find_child(root, b"\x01", C.byref(hit)) == -1
        assert lib._find_child(root, "日".encode()[:1], C.byref(hit)) >= 0     # a byte above 0x7f
        hand = Tok(root, None)
        libc = C.CDLL("libc.so.6")
        for text in (b"there and here", "日本語 ée".encode(), b"<|eot_id|>the abcd"):
            a, b = lib.tokenize(C.byref(hand), text), lib.tokenize(tk, text)
            assert [a[i] for i in range(a[0])] == [b[i] for i in range(b[0])]
            libc.free(a)
            libc.free(b)
    lib.free_tokenizer(tk, DECODE_SIZE)
