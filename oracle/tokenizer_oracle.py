"""CPU restatement of the reference tokenizer (src/tokenizer/tokenizer.cu:100-155): from each byte position
take the longest vocabulary string that matches, at most 2048 tokens; vocabulary entries first, added tokens
second, a repeated string keeps the id given last (tokenizer.cu:83-96, 275-298).

TEST INFRASTRUCTURE ONLY (pure Python, small cases): tests/ imports it, the product never does.
Pinned in tests/test_tokenizer.py by hand-worked examples, by a brute-force definition of "longest match"
and by the decode round trip."""
import json


def load_vocab(path):
    """bytes -> id as the trie holds them, and id -> bytes as the decode table holds them."""
    with open(path, "rb") as f:
        j = json.loads(f.read().decode("utf-8"))
    enc, dec = {}, {}
    for s, i in j["model"]["vocab"].items():
        b = s.encode("utf-8")
        if b"\0" in b:          # a C string ends at the first NUL (tokenizer.cu:279)
            b = b[:b.index(b"\0")]
        enc[b] = i
        dec[i] = b
    for e in j["added_tokens"]:
        b = e["content"].encode("utf-8")
        enc[b] = e["id"]
        dec[e["id"]] = b
    return enc, dec


def tokenize(enc, text_bytes, limit=2048):
    """Returns the ids, or raises ValueError(position) where the reference prints and exits."""
    longest = max(len(k) for k in enc)
    prefixes = set()
    for k in enc:
        for n in range(1, len(k) + 1):
            prefixes.add(k[:n])
    out, i = [], 0
    while i < len(text_bytes) and len(out) < limit:
        best, best_len = None, 0
        for n in range(1, min(longest, len(text_bytes) - i) + 1):
            piece = text_bytes[i:i + n]
            if piece not in prefixes:   # the trie walk stops at the first byte without a child (:125-128)
                break
            if piece in enc:
                best, best_len = enc[piece], n
        if best is None:
            raise ValueError(i)
        out.append(best)
        i += best_len
    return out
