"""Seeded synthetic tensors in the byte layouts the decode path consumes.

Everything here is plain numpy (``numpy.random.Generator(PCG64(seed))`` is
reproducible across machines), so the same buffers can be handed to the HIP
library and to any checker.

Layouts
-------
Q4_K super-block, 144 bytes / 256 weights (little-endian, no padding)::

    fp16 d @0 | fp16 dmin @2 | uint8 scales[12] @4 | uint8 qs[128] @16

``scales`` packs eight 6-bit sub-block scales and eight 6-bit mins; a weight
matrix ``W[N, K]`` is stored row by row, ``K/256`` blocks per row.

Q8_1 activation block, 36 bytes / 32 values, field order of the reference
(bench/bench.ts:6): ``int8 q[32] @0 | fp16 d @32 | fp16 s @34``.
"""
from __future__ import annotations

import numpy as np

Q4K_BLOCK_BYTES = 144
Q4K_BLOCK_ELEMS = 256
Q8_1_BLOCK_BYTES = 36
Q8_1_BLOCK_ELEMS = 32


def rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def f32_to_bf16(x) -> np.ndarray:
    """f32 -> bf16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def bf16_to_f32(h) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def pack_q4k_scales(sc: np.ndarray, m: np.ndarray) -> np.ndarray:
    """[..., 8] 6-bit scales and mins -> [..., 12] packed bytes."""
    sc = sc.astype(np.uint8)
    m = m.astype(np.uint8)
    out = np.empty(sc.shape[:-1] + (12,), np.uint8)
    out[..., 0:4] = (sc[..., 0:4] & 63) | ((sc[..., 4:8] >> 4) << 6)
    out[..., 4:8] = (m[..., 0:4] & 63) | ((m[..., 4:8] >> 4) << 6)
    out[..., 8:12] = (sc[..., 4:8] & 15) | ((m[..., 4:8] & 15) << 4)
    return out


def q4k_random(g: np.random.Generator, N: int, K: int, d_sigma: float = 0.01) -> np.ndarray:
    """Random Q4_K weight matrix, uint8 ``[N*K/256, 144]``.

    d, dmin = fp16(|N(0, d_sigma)|); sub-block scales and mins uniform 0..63;
    nibbles uniform 0..15.
    """
    if K % Q4K_BLOCK_ELEMS:
        raise ValueError(f"K={K} must be a multiple of 256")
    nblk = N * (K // Q4K_BLOCK_ELEMS)
    out = np.empty((nblk, Q4K_BLOCK_BYTES), np.uint8)
    dd = np.abs(g.standard_normal((nblk, 2), dtype=np.float32) * np.float32(d_sigma)).astype(np.float16)
    out[:, 0:4] = dd.view(np.uint8).reshape(nblk, 4)
    sc = g.integers(0, 64, (nblk, 8), dtype=np.uint8)
    mn = g.integers(0, 64, (nblk, 8), dtype=np.uint8)
    out[:, 4:16] = pack_q4k_scales(sc, mn)
    out[:, 16:144] = g.integers(0, 256, (nblk, 128), dtype=np.uint8)
    return out


def q4k_from_dense(w: np.ndarray) -> np.ndarray:
    """Quantize a dense f32 ``[N, K]`` matrix to Q4_K (simple min/max per sub-block).

    Used to build synthetic model weights whose dequantised values follow a chosen
    distribution; it is a generator of test data, not a reference quantizer.
    """
    N, K = w.shape
    if K % 256:
        raise ValueError("K must be a multiple of 256")
    sub = w.reshape(N, K // 256, 8, 32).astype(np.float32)
    mn = np.minimum(sub.min(-1), 0.0)
    mx = sub.max(-1)
    scale = (mx - mn) / 15.0                    # per sub-block step
    smin = -mn                                  # per sub-block offset (>= 0)
    d = (scale.max(-1) / 63.0).astype(np.float16)
    dmin = (smin.max(-1) / 63.0).astype(np.float16)
    df = d.astype(np.float32)[..., None]
    dmf = dmin.astype(np.float32)[..., None]
    sc = np.where(df > 0, np.rint(scale / np.where(df > 0, df, 1)), 0).clip(0, 63).astype(np.uint8)
    m = np.where(dmf > 0, np.rint(smin / np.where(dmf > 0, dmf, 1)), 0).clip(0, 63).astype(np.uint8)
    eff = df * sc.astype(np.float32)
    off = dmf * m.astype(np.float32)
    q = np.where(eff[..., None] > 0, np.rint((sub + off[..., None]) / np.where(eff > 0, eff, 1)[..., None]), 0)
    q = q.clip(0, 15).astype(np.uint8)         # [N, nb, 8, 32]
    nblk = N * (K // 256)
    out = np.empty((nblk, 144), np.uint8)
    out[:, 0:2] = d.reshape(nblk, 1).view(np.uint8)
    out[:, 2:4] = dmin.reshape(nblk, 1).view(np.uint8)
    out[:, 4:16] = pack_q4k_scales(sc.reshape(nblk, 8), m.reshape(nblk, 8))
    q = q.reshape(nblk, 4, 2, 32)
    out[:, 16:144] = (q[:, :, 0, :] | (q[:, :, 1, :] << 4)).reshape(nblk, 128)
    return out


def gemv_bytes(N: int, K: int, batch: int = 1) -> int:
    """Algorithmic HBM bytes of one Q4_K x Q8_1 GEMV: weights + Q8_1 x + f32 y."""
    return N * K * 144 // 256 + batch * (K // 32) * 36 + batch * N * 4


def paged_kv_random(g: np.random.Generator, B: int, L: int, NKV: int = 2, HD: int = 256,
                    page_size: int = 16, sigma: float = 1.0):
    """Paged bf16 KV cache for B sequences with lengths uniform in [L/2, L].

    Returns (kcache, vcache, block_table int32 [B, ceil(L/page)], ctx_len int32 [B]);
    caches are uint16 ``[num_pages, NKV, page_size, HD]`` and pages are handed out
    from a shuffled pool, so consecutive tokens are not consecutive in memory.
    """
    ctx = g.integers(L // 2, L + 1, B).astype(np.int32)
    ppseq = (L + page_size - 1) // page_size
    npages = B * ppseq
    pool = g.permutation(npages).astype(np.int32)
    bt = pool.reshape(B, ppseq)
    shape = (npages, NKV, page_size, HD)
    kc = f32_to_bf16(g.standard_normal(shape, dtype=np.float32) * np.float32(sigma))
    vc = f32_to_bf16(g.standard_normal(shape, dtype=np.float32) * np.float32(sigma))
    return kc, vc, bt, ctx


def q4k_centered(g: np.random.Generator, N: int, K: int, sigma: float) -> np.ndarray:
    """Random Q4_K matrix whose dequantised weights are zero-mean with standard deviation ~sigma.

    Per super-block: sub-block scales uniform in 8..31, mins = round(7.5/8 * scale) with
    dmin = 8*d, so that w = d*sc*nib - dmin*m ~ d*sc*(nib - 7.5); d is drawn around
    sigma / (4.61 * 19.5) (4.61 = std of a uniform nibble, 19.5 = mean scale).
    Used for the synthetic model: random-nibble blocks with independent mins have a large
    common offset per row, which no trained or initialised model has.
    """
    if K % Q4K_BLOCK_ELEMS:
        raise ValueError(f"K={K} must be a multiple of 256")
    nblk = N * (K // Q4K_BLOCK_ELEMS)
    out = np.empty((nblk, Q4K_BLOCK_BYTES), np.uint8)
    d = (sigma / (4.61 * 19.5)) * (0.5 + g.random(nblk, dtype=np.float32))
    dd = np.stack([d, 8.0 * d], axis=1).astype(np.float16)
    out[:, 0:4] = dd.view(np.uint8).reshape(nblk, 4)
    sc = g.integers(8, 32, (nblk, 8), dtype=np.uint8)
    mn = np.rint(sc.astype(np.float32) * (7.5 / 8.0)).astype(np.uint8)
    out[:, 4:16] = pack_q4k_scales(sc, mn)
    out[:, 16:144] = g.integers(0, 256, (nblk, 128), dtype=np.uint8)
    return out
