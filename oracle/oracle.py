"""ctypes front-end of the CPU oracle (``liboracle.so``, built from ``oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()``
and by the CPU-baseline leg of ``bench.py``; never by the shipped package.

bf16 and fp16 tensors are passed as ``numpy.uint16`` bit patterns, Q4_K / Q8_1
data as ``numpy.uint8`` byte arrays.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force: bool = False) -> str:
    """Compile oracle.c with gcc (``make -C oracle``)."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "oracle.c"))
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_encode_half.restype = C.c_uint16
        _lib.orc_encode_half.argtypes = [C.c_double]
        _lib.orc_half_to_float.restype = C.c_float
        _lib.orc_half_to_float.argtypes = [C.c_uint16]
        _lib.orc_half_to_float_ftz.restype = C.c_float
        _lib.orc_half_to_float_ftz.argtypes = [C.c_uint16]
        _lib.orc_f32_to_bf16.restype = C.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [C.c_float]
        _lib.orc_f32_to_half_rne.restype = C.c_uint16
        _lib.orc_f32_to_half_rne.argtypes = [C.c_float]
    return _lib


def set_threads(n: int) -> None:
    """OpenMP threads of the row / head loops from now on."""
    lib().orc_set_threads(int(n))


def max_threads() -> int:
    return int(lib().orc_max_threads())


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


# ---------------------------------------------------------------- conversions
def encode_half(v: float) -> int:
    return int(lib().orc_encode_half(float(v)))


def half_to_float(h: int) -> float:
    return float(lib().orc_half_to_float(int(h)))


def half_to_float_ftz(h: int) -> float:
    return float(lib().orc_half_to_float_ftz(int(h)))


def f32to16(x) -> np.ndarray:
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().orc_f32to16(_p(x), _p(out), C.c_int64(x.size))
    return out


def f32_to_bf16(x) -> np.ndarray:
    """Round-to-nearest-even f32 -> bf16 bit patterns (vectorised, same rule as the C helper)."""
    u = _c(x, np.float32).view(np.uint32).astype(np.uint64)
    nan = ((u & 0x7F800000) == 0x7F800000) & ((u & 0x7FFFFF) != 0)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_to_f32(h) -> np.ndarray:
    return (_c(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---------------------------------------------------------------- Q8_1
def pack_q8_1(x) -> np.ndarray:
    x = _c(x, np.float32).ravel()
    nb = (x.size + 31) // 32
    out = np.zeros(nb * 36, np.uint8)
    lib().orc_pack_q8_1(_p(x), C.c_int64(x.size), _p(out))
    return out


def pack_q8_1_rows(x) -> np.ndarray:
    """Quantize each row of a [B, K] array; returns uint8 [B, K/32*36]."""
    x = _c(x, np.float32)
    return np.stack([pack_q8_1(r) for r in x.reshape(-1, x.shape[-1])])


# ---------------------------------------------------------------- legacy block
def legacy_dequant_i8(blocks) -> np.ndarray:
    blocks = _c(blocks, np.uint8).ravel()
    nb = blocks.size // 20
    out = np.empty(nb * 32, np.int8)
    lib().orc_legacy_dequant_i8(_p(blocks), C.c_int64(nb), _p(out))
    return out


def legacy_pack_q4k_col(data, K, N) -> np.ndarray:
    data = _c(data, np.float32)
    nb = (K + 31) // 32
    out = np.zeros(N * nb * 20, np.uint8)
    lib().orc_legacy_pack_q4k_col(_p(data), K, N, _p(out))
    return out


def legacy_qmm(A, B, M, N, K) -> np.ndarray:
    A = _c(A, np.uint8); B = _c(B, np.uint8)
    out = np.empty((M, N), np.float32)
    lib().orc_legacy_qmm(_p(A), _p(B), _p(out), M, N, K)
    return out


def i8_gemm(A, B) -> np.ndarray:
    A = _c(A, np.int8); B = _c(B, np.int8)
    M, K = A.shape; K2, N = B.shape
    assert K == K2
    out = np.empty((M, N), np.int32)
    lib().orc_i8_gemm(_p(A), _p(B), _p(out), M, N, K)
    return out


# ---------------------------------------------------------------- Q4_K super-block
def q4k_unpack_scales(scales12):
    s = _c(scales12, np.uint8)
    sc = np.empty(8, np.uint8); m = np.empty(8, np.uint8)
    lib().orc_q4k_unpack_scales(_p(s), _p(sc), _p(m))
    return sc, m


def q4k_pack_scales(sc, m) -> np.ndarray:
    sc = _c(sc, np.uint8); m = _c(m, np.uint8)
    out = np.empty(12, np.uint8)
    lib().orc_q4k_pack_scales(_p(sc), _p(m), _p(out))
    return out


def q4k_nibbles(blocks) -> np.ndarray:
    blocks = _c(blocks, np.uint8).ravel()
    nb = blocks.size // 144
    out = np.empty(nb * 256, np.uint8)
    lib().orc_q4k_nibbles(_p(blocks), C.c_int64(nb), _p(out))
    return out


def q4k_dequant(blocks) -> np.ndarray:
    blocks = _c(blocks, np.uint8).ravel()
    nb = blocks.size // 144
    out = np.empty(nb * 256, np.float32)
    lib().orc_q4k_dequant(_p(blocks), C.c_int64(nb), _p(out))
    return out


def f32_to_half_rne(v: float) -> int:
    return int(lib().orc_f32_to_half_rne(float(v)))


def qkx2_fit32(x, weights):
    """(scale, the_min, L[32]) of one 32-element sub-block."""
    x = _c(x, np.float32); weights = _c(weights, np.float32)
    assert x.size == 32 and weights.size == 32
    L = np.zeros(32, np.uint8); the_min = C.c_float(0)
    f = lib().orc_qkx2_fit32
    f.restype = C.c_float
    scale = f(_p(x), _p(weights), _p(L), C.byref(the_min))
    return float(scale), float(the_min.value), L


def quantize_q4k(x) -> np.ndarray:
    """f32 values (a multiple of 256 of them, row-major weights) -> 144-byte super-blocks."""
    x = _c(x, np.float32).ravel()
    assert x.size % 256 == 0
    out = np.zeros(x.size // 256 * 144, np.uint8)
    lib().orc_quantize_q4k(_p(x), C.c_int64(x.size), _p(out))
    return out


def gemv_q4k_f32(W, x, N, K, acc64=True) -> np.ndarray:
    W = _c(W, np.uint8); x = _c(x, np.float32)
    y = np.empty(N, np.float32)
    lib().orc_gemv_q4k_f32(_p(W), _p(x), _p(y), N, K, int(acc64))
    return y


def q4k_q8_1_subdots(W, xq, N, K) -> np.ndarray:
    W = _c(W, np.uint8); xq = _c(xq, np.uint8)
    out = np.empty((N, K // 32), np.int32)
    lib().orc_q4k_q8_1_subdots(_p(W), _p(xq), _p(out), N, K)
    return out


def gemv_q4k_q8_1(W, xq, N, K, acc64=True) -> np.ndarray:
    W = _c(W, np.uint8); xq = _c(xq, np.uint8)
    y = np.empty(N, np.float32)
    lib().orc_gemv_q4k_q8_1(_p(W), _p(xq), _p(y), N, K, int(acc64))
    return y


# ---------------------------------------------------------------- glue
def embed(E, token, H) -> np.ndarray:
    E = _c(E, np.uint16)
    out = np.empty(H, np.uint16)
    lib().orc_embed(_p(E), int(token), _p(out), H)
    return out


def rmsnorm(x, w) -> np.ndarray:
    x = _c(x, np.uint16); w = _c(w, np.uint16)
    out = np.empty(x.size, np.uint16)
    lib().orc_rmsnorm(_p(x), _p(w), _p(out), x.size)
    return out


def cast_bf16(x) -> np.ndarray:
    x = _c(x, np.float32)
    out = np.empty(x.size, np.uint16)
    lib().orc_cast_bf16(_p(x), _p(out), x.size)
    return out


def add_bf16(a, b) -> np.ndarray:
    a = _c(a, np.uint16); b = _c(b, np.uint16)
    out = np.empty(a.size, np.uint16)
    lib().orc_add_bf16(_p(a), _p(b), _p(out), a.size)
    return out


def swiglu(g, u) -> np.ndarray:
    g = _c(g, np.float32); u = _c(u, np.float32)
    out = np.empty(g.size, np.uint16)
    lib().orc_swiglu(_p(g), _p(u), _p(out), g.size)
    return out


def conv1d_decode(x, st, w):
    x = _c(x, np.uint16); st = _c(st, np.uint16); w = _c(w, np.uint16)
    Cn = x.size
    out = np.empty(Cn, np.uint16); stn = np.empty(3 * Cn, np.uint16)
    lib().orc_conv1d_decode(_p(x), _p(st), _p(w), _p(out), _p(stn), Cn)
    return out, stn.reshape(3, Cn)


def headnorm(x, w, nheads, HD, in_stride) -> np.ndarray:
    x = _c(x, np.uint16); w = _c(w, np.uint16)
    out = np.empty(nheads * HD, np.uint16)
    lib().orc_headnorm(_p(x), _p(w), _p(out), nheads, HD, in_stride)
    return out


def rope_tables(max_len, rot_dim=64, theta=1e7):
    half = rot_dim // 2
    c = np.empty((max_len, half), np.float32); s = np.empty((max_len, half), np.float32)
    lib().orc_rope_tables(_p(c), _p(s), max_len, rot_dim, C.c_double(theta))
    return c, s


def rope(x, cos_t, sin_t, pos, nheads, HD, half=32) -> np.ndarray:
    x = np.array(_c(x, np.uint16), copy=True)
    cos_t = _c(cos_t, np.float32); sin_t = _c(sin_t, np.float32)
    lib().orc_rope(_p(x), _p(cos_t), _p(sin_t), int(pos), nheads, HD, half)
    return x


def argmax(logits):
    logits = _c(logits, np.float32).ravel()
    v = C.c_float(); i = C.c_int32()
    lib().orc_argmax(_p(logits), C.c_int64(logits.size), C.byref(v), C.byref(i))
    return float(v.value), int(i.value)


# ---------------------------------------------------------------- GDN
def gdn_step(conv_out, z, A_log, dt_bias, a_p, b_p, norm_w, S, Hg, dk=128, dv=128, rows_per_chain=16):
    conv_out = _c(conv_out, np.uint16); z = _c(z, np.uint16)
    A_log = _c(A_log, np.float32); dt_bias = _c(dt_bias, np.uint16)
    a_p = _c(a_p, np.float32); b_p = _c(b_p, np.float32); norm_w = _c(norm_w, np.float32)
    S = _c(S, np.float32)
    out = np.empty(Hg * dv, np.uint16); Sn = np.empty(Hg * dk * dv, np.float32)
    lib().orc_gdn_step(_p(conv_out), _p(z), _p(A_log), _p(dt_bias), _p(a_p), _p(b_p), _p(norm_w),
                       _p(S), _p(out), _p(Sn), Hg, dk, dv, int(rows_per_chain))
    return out, Sn.reshape(Hg, dk, dv)


def gdn_core(q, k, v, g, beta, S, Hg, dk=128, dv=128):
    q = _c(q, np.uint16); k = _c(k, np.uint16); v = _c(v, np.uint16)
    g = _c(g, np.float32); beta = _c(beta, np.float32); S = _c(S, np.float32)
    out = np.empty(Hg * dv, np.uint16); Sn = np.empty(Hg * dk * dv, np.float32)
    lib().orc_gdn_core(_p(q), _p(k), _p(v), _p(g), _p(beta), _p(S), _p(out), _p(Sn), Hg, dk, dv)
    return out, Sn.reshape(Hg, dk, dv)


# ---------------------------------------------------------------- attention
def attn_decode_paged(q, kc, vc, block_table, ctx_len, B, NH, NKV, HD, page_size=16,
                      gate=None, gate_bstride=0, gate_hstride=0):
    q = _c(q, np.uint16); kc = _c(kc, np.uint16); vc = _c(vc, np.uint16)
    bt = _c(block_table, np.int32).reshape(B, -1); cl = _c(ctx_len, np.int32)
    g = _c(gate, np.uint16) if gate is not None else None
    out = np.empty((B, NH, HD), np.uint16); lse = np.empty((B, NH), np.float32)
    lib().orc_attn_decode_paged(_p(q), _p(kc), _p(vc), _p(bt), bt.shape[1], _p(cl),
                                _p(g), int(gate_bstride), int(gate_hstride),
                                _p(out), _p(lse), B, NH, NKV, HD, page_size)
    return out, lse


def kv_append(k, v, kc, vc, block_table, pos, NKV, HD, page_size=16):
    """In-place write of one token's k, v into the paged caches (numpy uint16 arrays)."""
    k = _c(k, np.uint16); v = _c(v, np.uint16)
    bt = _c(block_table, np.int32)
    assert kc.flags.c_contiguous and vc.flags.c_contiguous and kc.dtype == np.uint16
    lib().orc_kv_append(_p(k), _p(v), _p(kc), _p(vc), _p(bt), int(pos), NKV, HD, page_size)
