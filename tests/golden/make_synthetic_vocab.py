"""Writes tests/golden/synthetic_vocab.txt: a small vocabulary in the RWKV "world" file format.

Each line is `<id> <repr of a Python str or bytes object> <length in bytes>`.  Ids 1..256 are the single
bytes 0..255 (as in the real vocabulary, so id = byte + 1: 'o','p','q' are 112,113,114); bytes that are
valid one-byte UTF-8 are written as str, the rest as bytes.  Longer tokens follow: English fragments, CJK
characters, an emoji, and a few partial UTF-8 sequences as bytes tokens so that a token boundary can fall
inside a character.  The file is data for the tokenizer/engine tests; it is not derived from the real
vocabulary file.

    python tests/golden/make_synthetic_vocab.py
"""
import os

WORDS = [
    "\n\n", "\t\t", "  ", "    ", ": ", ", ", ". ", "th", "he", "in", "er", "an", "re", "on", "at", "en", "is",
    "es", "st", " a", " t", " s", " i", " th", "the", " the", "ing", "and", " and", " is", " test", "test",
    " answer", "answer", "This", " This", "User", "Assistant", "System", "User:", "Assistant:", "System:",
    "prompt", "round", "trip", "hi", " hi", "extra", "<think", "</think", "think", " (think", " a bit)",
    "It's", "\\n", "'quoted'", '"', "'\"", "0123456789", " " * 16,
    "中", "文", "中文", "你好", "世界", "嗯", "日本語", "テスト", "é", "ü", "é\n", "😀", "👍🏽",
]
BYTES = [b"\xe4\xb8", b"\xe4", b"\xf0\x9f", b"\xf0\x9f\x98", b"\xff\xfe", b"\xc3"]


def main():
    out = []
    tid = 1
    for b in range(256):
        raw = bytes([b])
        obj = raw.decode("utf-8") if b < 0x80 else raw
        out.append("%d %r %d" % (tid, obj, 1))
        tid += 1
    seen = set()
    for w in WORDS:
        raw = w.encode("utf-8")
        if len(raw) < 2 or raw in seen:
            continue
        seen.add(raw)
        out.append("%d %r %d" % (tid, w, len(raw)))
        tid += 1
    for raw in BYTES:
        if len(raw) < 2 or raw in seen:
            continue
        seen.add(raw)
        out.append("%d %r %d" % (tid, raw, len(raw)))
        tid += 1
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "synthetic_vocab.txt")
    with open(path, "w", encoding="utf-8", newline="\n") as f:
        f.write("\n".join(out) + "\n")
    print("wrote", path, len(out), "tokens")


if __name__ == "__main__":
    main()
