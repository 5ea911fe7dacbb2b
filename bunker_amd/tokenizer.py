"""Text -> token ids through ``libbunker_tok.so`` (``gt_init`` / ``gt_encode`` / ``gt_encode_mt`` / ``gt_free``), the C ABI the reference
binds for its tokenizer (prototypes/decode.ts:78-86 over shim/gigatoken_wrapper/src/lib.rs:19-93)."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libbunker_tok.so")
_lib = None


def load_library():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `make -C bunker_amd/tok`")
        lib = C.CDLL(LIB_PATH)
        lib.gt_init.restype = C.c_void_p
        lib.gt_init.argtypes = [C.c_char_p]
        lib.gt_encode.restype = C.c_int
        lib.gt_encode.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, C.c_void_p, C.c_size_t]
        lib.gt_encode_mt.restype = C.c_int
        lib.gt_encode_mt.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, C.c_void_p, C.c_size_t]
        lib.gt_free.restype = None
        lib.gt_free.argtypes = [C.c_void_p]
        lib.gt_last_error.restype = C.c_char_p
        lib.gt_last_error.argtypes = []
        _lib = lib
    return _lib


class Tokenizer:
    def __init__(self, tok_path: str):
        lib = load_library()
        self.h = lib.gt_init(tok_path.encode("utf-8"))
        if not self.h:
            raise RuntimeError("gt_init failed: " + lib.gt_last_error().decode("utf-8", "replace"))

    def encode(self, text: str | bytes, mt: bool = False) -> np.ndarray:
        """``mt``: gt_encode_mt (prototypes/gigatoken_bun.ts:30) — the text cut at spaces into one chunk per hardware
        thread and the chunks encoded side by side."""
        data = text.encode("utf-8") if isinstance(text, str) else bytes(text)
        out = np.empty(len(data) + 64, np.uint32)            # decode.ts:82: at most one id per byte
        fn = load_library().gt_encode_mt if mt else load_library().gt_encode
        rc = fn(self.h, data, len(data), out.ctypes.data_as(C.c_void_p), out.size)
        if rc < 0:
            raise RuntimeError("gt_encode failed")
        return out[:rc].copy()

    def close(self) -> None:
        if self.h:
            load_library().gt_free(self.h)
            self.h = None


def tokenize(text: str, tok_path: str) -> np.ndarray:
    """prototypes/decode.ts:78-86: open the tokenizer, encode, close."""
    t = Tokenizer(tok_path)
    try:
        return t.encode(text)
    finally:
        t.close()
