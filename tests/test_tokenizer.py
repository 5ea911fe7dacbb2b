"""The C++ byte-level BPE behind gt_init / gt_encode / gt_free against the Hugging Face `tokenizers` library (the
published implementation of the tokenizer.json format) on the same file: a small vocabulary trained here on this
repository's own documents, with the pre-tokenizer expression of the Qwen family (one digit per piece) and of the
cl100k family (up to three)."""
import os

import numpy as np
import pytest

tokenizers = pytest.importorskip("tokenizers")

from bunker_amd import tokenizer

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
QWEN = r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+"
CL100K = r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}{1,3}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+"
SPECIAL = ["<|endoftext|>", "<|im_start|>", "<|im_end|>", "<|im_start|>assistant"]


def _train(path, pattern, ignore_merges=False):
    from tokenizers import Regex, Tokenizer, decoders, models, pre_tokenizers, trainers
    tok = Tokenizer(models.BPE(ignore_merges=ignore_merges))
    tok.pre_tokenizer = pre_tokenizers.Sequence([pre_tokenizers.Split(Regex(pattern), behavior="isolated", invert=False),
                                                 pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)])
    tok.decoder = decoders.ByteLevel()
    tr = trainers.BpeTrainer(vocab_size=3000, special_tokens=SPECIAL, initial_alphabet=pre_tokenizers.ByteLevel.alphabet(),
                             show_progress=False)
    text = open(os.path.join(ROOT, "README.md")).read() + open(os.path.join(ROOT, "bunker_amd", "runner.py")).read()
    text += open(os.path.join(ROOT, "bunker_amd", "loader.py")).read()
    text += " 日本語のテキスト 한국어 텍스트 naïve café 12345 67 890 😀 " * 20
    tok.train_from_iterator([text[i:i + 1500] for i in range(0, len(text), 1500)], tr)
    tok.save(path)
    return tok


FIXED = ["", " ", "  ", "\n", "a", "Hello world's  12345 <|im_start|>x\n\n  y", "I'm we'LL they'Re 'd 'S 'T", "don't can't WON'T",
         "x = y+z; // comment\r\n\r\n\tindent", "日本語のテキスト と 한국어 123४५", "tabs\t\t!\n", "   \n   \n", "end with spaces   ",
         "naïve café ÀÉ", "emoji 😀😀 ok", "<|endoftext|><|im_end|>", "a<|im_start|", "<|im_start|>assistant\nhi<|im_end|>",
         "1234567890 3.14159 1,000,000", " nbsp x　wide em", "ⅷ ½ ² ٣", "_under_score __init__", "a\r\nb\rc\n\nd",
         "\t\t\tx", "x \n y", "  5", " !?", "...\n\n\n", "é combining", "﻿bom"]


def _fuzz(rng, n):
    pools = ["abcXYZ", "0123456789", " \t\n\r", " ", ".,;:!?'\"()[]{}<>|/\\-_=+*&^%$#@~`", "日本語한국어", "éüßñ", "😀🙂", "٣४ⅷ½",
             " 　 ", "'s't're've'm'll'd"]
    out = []
    for _ in range(n):
        parts = []
        for _ in range(int(rng.integers(1, 12))):
            pool = pools[int(rng.integers(0, len(pools)))]
            parts.append("".join(pool[int(i)] for i in rng.integers(0, len(pool), int(rng.integers(1, 6)))))
            if rng.random() < 0.05:
                parts.append(SPECIAL[int(rng.integers(0, len(SPECIAL)))])
        out.append("".join(parts))
    return out


@pytest.mark.parametrize("pattern,ignore_merges", [(QWEN, False), (CL100K, False), (QWEN, True)])
def test_encode_equals_hugging_face(tmp_path, pattern, ignore_merges):
    path = str(tmp_path / "tokenizer.json")
    hf = _train(path, pattern, ignore_merges)
    t = tokenizer.Tokenizer(path)
    docs = [open(os.path.join(ROOT, "bunker_amd", "model.py")).read(), open(os.path.join(ROOT, "bench.py")).read()[:20000]]
    for s in FIXED + _fuzz(np.random.default_rng(7), 600) + docs:
        got, ref = t.encode(s).tolist(), hf.encode(s).ids
        assert got == ref, (s[:80], got[:16], ref[:16])
    t.close()
    assert tokenizer.tokenize("Hello", path).tolist() == hf.encode("Hello").ids


def test_repeated_pieces_and_the_bounds_of_the_piece_table(tmp_path):
    """encode keeps the ids of pieces of up to 24 bytes and 8 ids for the rest of the call: pieces at and past both
    bounds, seen twice in one call and between other pieces that land in the same table, give the Hugging Face ids."""
    path = str(tmp_path / "tokenizer.json")
    hf = _train(path, QWEN)
    t = tokenizer.Tokenizer(path)
    rng = np.random.default_rng(11)
    words = []
    for n in (1, 7, 8, 9, 23, 24, 25, 40):
        words.append("".join("qzxjkvw"[int(i)] for i in rng.integers(0, 7, n)))            # rare letters: about one id a byte
        words.append(("tokenizer" * 5)[:n])                                                 # common letters: few ids
    words += ["日本語한국어日本", "😀🙂😀🙂😀🙂"]                                            # 24 bytes of 3- and 4-byte characters
    filler = [f"w{i}" for i in range(40000)]                                                 # more pieces than the table has slots
    text = " ".join(words) + " " + " ".join(filler) + " " + " ".join(reversed(words)) + SPECIAL[0] + " ".join(words)
    assert t.encode(text).tolist() == hf.encode(text).ids
    t.close()


def test_abi_errors_and_truncation(tmp_path):
    import ctypes as C
    lib = tokenizer.load_library()
    assert not lib.gt_init(b"/nonexistent/tokenizer.json") and b"cannot open" in lib.gt_last_error()
    bad = tmp_path / "bad.json"; bad.write_text("{\"model\": {\"type\": \"BPE\"}}")
    assert not lib.gt_init(str(bad).encode()) and b"model.vocab" in lib.gt_last_error()
    path = str(tmp_path / "tokenizer.json")
    hf = _train(path, QWEN)
    h = lib.gt_init(path.encode())
    assert h
    out = np.zeros(3, np.uint32)
    text = b"one two three four five"
    assert lib.gt_encode(h, text, len(text), out.ctypes.data_as(C.c_void_p), 3) == 3           # at most out_max ids
    assert out.tolist() == hf.encode(text.decode()).ids[:3]
    assert lib.gt_encode(None, text, len(text), out.ctypes.data_as(C.c_void_p), 3) == -1
    lib.gt_free(h)


def _mt_chunks(data: bytes, n_threads: int):
    """The cuts of shim/gigatoken_wrapper/src/lib.rs:55-63: equal shares of the bytes, each run on to just behind the next space."""
    size = (len(data) + n_threads - 1) // n_threads
    out, s = [], 0
    while s < len(data):
        e = min(s + size, len(data))
        if e < len(data):
            while e < len(data) and data[e] != 0x20:
                e += 1
            if e < len(data):
                e += 1
        out.append(data[s:e])
        s = e
    return out


def test_encode_mt_is_encode_over_space_cut_chunks(tmp_path):
    import ctypes as C
    path = str(tmp_path / "tokenizer.json")
    hf = _train(path, QWEN)
    t = tokenizer.Tokenizer(path)
    n_threads = os.cpu_count() or 32
    docs = [open(os.path.join(ROOT, "bench.py")).read(), "no-spaces-at-all" * 50, "", "a", "a b", " 日本語 한국어 😀 " * 300]
    for s in docs:
        data = s.encode("utf-8")
        want = [i for c in _mt_chunks(data, n_threads) for i in hf.encode(c.decode("utf-8", "ignore")).ids] \
            if all(_valid_utf8(c) for c in _mt_chunks(data, n_threads)) else None
        got = t.encode(s, mt=True).tolist()
        assert got == [i for c in _mt_chunks(data, n_threads) for i in t.encode(c).tolist()], s[:40]
        if want is not None:
            assert got == want, s[:40]
    # a text without spaces is one chunk per share run to the end: the same ids as the single-thread call
    assert t.encode("no-spaces-at-all" * 50, mt=True).tolist() == t.encode("no-spaces-at-all" * 50).tolist()
    # the count returned is the total even when it exceeds out_max; chunks that do not fit are left out
    lib = tokenizer.load_library()
    text = ("word " * 400).encode()
    full = t.encode(text, mt=True)
    small = np.full(5, 0xFFFFFFFF, np.uint32)
    assert lib.gt_encode_mt(t.h, text, len(text), small.ctypes.data_as(C.c_void_p), 5) == len(full)
    assert lib.gt_encode_mt(None, text, len(text), small.ctypes.data_as(C.c_void_p), 5) == -1
    t.close()


def _valid_utf8(b: bytes) -> bool:
    try:
        b.decode("utf-8")
        return True
    except UnicodeDecodeError:
        return False
