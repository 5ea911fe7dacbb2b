"""Pins the oracle's quantization functions with checks that do not reuse its formulas:
known answers from the reference's own tests, exhaustive fp16 sweeps against numpy's
IEEE half type, hand-computed blocks and integer special cases."""
import numpy as np
import pytest

from bunker_amd import synth


# ------------------------------------------------------------------ fp16
def test_encode_half_hand_vectors(orc):
    # bench/bench.ts:41-51: truncation, flush below 2^-14, Inf at and above 2^16
    assert orc.encode_half(0.0) == 0
    assert orc.encode_half(1.0) == 0x3C00
    assert orc.encode_half(-2.0) == 0xC000
    assert orc.encode_half(65504.0) == 0x7BFF
    assert orc.encode_half(65519.99) == 0x7BFF          # RNE would already be Inf at 65520
    assert orc.encode_half(65536.0) == 0x7C00
    assert orc.encode_half(-1e9) == 0xFC00
    assert orc.encode_half(6.0e-5) == 0                   # below the smallest normal 6.1035e-5
    assert orc.encode_half(-6.0e-5) == 0x8000
    assert orc.encode_half(2.0 ** -14) == 0x0400
    # 1 + 2^-10 + 2^-11 : the dropped bit must not round up
    assert orc.encode_half(1.0 + 2.0 ** -10 + 2.0 ** -11) == 0x3C01
    assert orc.encode_half(1.0 + 2.0 ** -10 - 2.0 ** -20) == 0x3C00


def test_encode_half_is_truncation_everywhere(orc):
    g = synth.rng(1)
    x = np.concatenate([g.standard_normal(20000) * 10.0 ** g.integers(-4, 5, 20000), [0.1, 0.3, 1e-3]])
    x32 = x.astype(np.float32)
    got = np.array([orc.encode_half(float(v)) for v in x], np.uint16)
    dec = got.view(np.float16).astype(np.float64)
    a = np.abs(x32.astype(np.float64))
    normal = (a >= 2.0 ** -14) & (a < 65536.0)
    # truncation: |dec| <= |x| < |dec| + ulp, same sign
    ulp = 2.0 ** (np.floor(np.log2(np.where(normal, a, 1.0))) - 10)
    assert np.all(np.abs(dec[normal]) <= a[normal])
    assert np.all(a[normal] - np.abs(dec[normal]) < ulp[normal])
    assert np.all(np.sign(dec[normal]) == np.sign(x32[normal]))
    assert np.all(np.abs(dec[a < 2.0 ** -14]) == 0)


def test_fp16_exhaustive_round_trip(orc):
    h = np.arange(65536, dtype=np.uint16)
    ref = h.view(np.float16).astype(np.float32)            # numpy's exact IEEE decode
    got = np.array([orc.half_to_float(int(v)) for v in h], np.float32)
    finite = np.isfinite(ref)
    assert np.array_equal(got[finite], ref[finite])
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.array_equal(np.isinf(got), np.isinf(ref))
    # encode(decode(h)) == h for every normal number; denormals flush to signed zero
    e = (h >> 10) & 31
    normal = (e > 0) & (e < 31)
    enc = np.array([orc.encode_half(float(v)) for v in ref[normal]], np.uint16)
    assert np.array_equal(enc, h[normal])
    den = (e == 0) & ((h & 0x3FF) != 0)
    enc_d = np.array([orc.encode_half(float(v)) for v in ref[den]], np.uint16)
    assert np.array_equal(enc_d, h[den] & 0x8000)
    # the vectorised variant (src/kernel.ts:16-32) agrees on all finite inputs
    assert np.array_equal(orc.f32to16(ref[normal]), h[normal])
    assert np.array_equal(orc.f32to16(ref[den]), h[den] & 0x8000)
    assert orc.f32to16(np.array([np.inf, -np.inf], np.float32)).tolist() == [0x7C00, 0xFC00]
    assert orc.f32to16(np.array([np.nan], np.float32))[0] & 0x7E00 == 0x7E00


def test_half_to_float_ftz(orc):
    # src/dsl.ts:955-975: exponent field 0 -> +0.0, otherwise the plain bit shuffle
    assert orc.half_to_float_ftz(0x0001) == 0.0
    assert orc.half_to_float_ftz(0x83FF) == 0.0
    assert orc.half_to_float_ftz(0x3C00) == 1.0
    assert orc.half_to_float_ftz(0xC000) == -2.0
    h = np.arange(0x0400, 0x7C00, 7, dtype=np.uint16)
    got = np.array([orc.half_to_float_ftz(int(v)) for v in h], np.float32)
    assert np.array_equal(got, h.view(np.float16).astype(np.float32))


def test_bf16_round_to_nearest_even(orc):
    f = np.array([1.0, 1.0 + 2 ** -8, 1.0 + 2 ** -7 + 2 ** -8, 1.0 + 2 ** -8 + 2 ** -20, -3.5, 0.0], np.float32)
    # ties go to the even mantissa: 1+2^-8 -> 1.0 ; 1+2^-7+2^-8 -> 1+2^-6
    exp = [0x3F80, 0x3F80, 0x3F82, 0x3F81, 0xC060, 0x0000]
    assert orc.f32_to_bf16(f).tolist() == exp
    assert [orc.lib().orc_f32_to_bf16(float(v)) for v in f] == exp
    assert synth.f32_to_bf16(f).tolist() == exp
    x = synth.rng(2).standard_normal(1000).astype(np.float32)
    assert np.array_equal(orc.f32_to_bf16(x), synth.f32_to_bf16(x))


# ------------------------------------------------------------------ Q8_1
def _q8_fields(buf):
    b = buf.reshape(-1, 36)
    q = b[:, :32].view(np.int8)
    d = b[:, 32:34].copy().view(np.float16).astype(np.float64).ravel()
    s = b[:, 34:36].copy().view(np.float16).astype(np.float64).ravel()
    return q, d, s


def test_q8_1_ties_round_toward_plus_infinity(orc):
    # amax = 127 makes d exactly 1, so x/d is x: JS Math.round semantics are visible
    x = np.zeros(32, np.float32)
    x[0] = 127.0
    x[1:9] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.49999997, -0.50000006]
    q, d, s = _q8_fields(orc.pack_q8_1(x))
    assert d[0] == 1.0
    assert q[0, :9].tolist() == [127, 1, 0, 2, -1, 3, -2, 0, -1]
    assert s[0] == float(sum([127, 1, 0, 2, -1, 3, -2, 0, -1]))


def test_q8_1_properties(orc):
    g = synth.rng(3)
    x = g.standard_normal(32 * 257).astype(np.float32)
    x[32:64] = 0.0                                         # an all-zero block
    q, d, s = _q8_fields(orc.pack_q8_1(x))
    xb = x.reshape(-1, 32).astype(np.float64)
    amax = np.abs(xb).max(1)
    dt = amax / 127.0                                      # unrounded d used for the quotient
    assert np.all(np.abs(xb - dt[:, None] * q) <= dt[:, None] / 2 * (1 + 1e-12))
    nz = amax > 0
    assert np.all(np.abs(q[nz]).max(1) == 127)
    assert np.all(q[~nz] == 0) and np.all(d[~nz] == 0) and np.all(s[~nz] == 0)
    # stored d is the truncated fp16 of amax/127 (never above it, within one fp16 ulp)
    assert np.all(d <= dt) and np.all(dt - d < dt * 2.0 ** -10 + 1e-30)
    # stored s is trunc16(sum(q) * unrounded d)
    st = q.astype(np.int64).sum(1) * dt
    assert np.all(np.abs(s) <= np.abs(st) + 1e-30)
    assert np.all(np.abs(st - s) <= np.abs(st) * 2.0 ** -10 + 2.0 ** -14)


def test_q8_1_ragged_tail(orc):
    x = np.arange(1, 41, dtype=np.float32)                 # 40 elements -> 2 blocks, 24 pad
    buf = orc.pack_q8_1(x)
    assert buf.size == 72
    q, d, s = _q8_fields(buf)
    assert np.all(q[1, 8:] == 0)
    assert q[1, 7] == 127 and q[0, 31] == 127


# ------------------------------------------------------------------ legacy 20-byte block
def test_legacy_dequant_known_answer(orc):
    # tests/test_dequant.ts:13-24: byte = lo | hi<<4  ->  [lo-8, hi-8] interleaved
    g = synth.rng(4)
    nb = 128 * 32
    lo = g.integers(0, 16, (nb, 16)); hi = g.integers(0, 16, (nb, 16))
    blocks = np.zeros((nb, 20), np.uint8)
    blocks[:, :16] = lo | (hi << 4)
    ref = np.empty((nb, 32), np.int8)
    ref[:, 0::2] = lo - 8
    ref[:, 1::2] = hi - 8
    assert np.array_equal(orc.legacy_dequant_i8(blocks), ref.ravel())


def test_i8_gemm_exact(orc):
    # tests/test_q4k_pipeline.ts:111-116 triple loop == exact integer matmul
    g = synth.rng(5)
    A = g.integers(-8, 8, (32, 1024)).astype(np.int8)
    B = g.integers(-128, 128, (1024, 32)).astype(np.int8)
    assert np.array_equal(orc.i8_gemm(A, B), A.astype(np.int64) @ B.astype(np.int64))


def test_legacy_qmm_against_float_dot(orc):
    # bench/bench.ts:10-38 with w = d*q + dmin and x ~ d8*q8: compare with a float64 dot
    g = synth.rng(6)
    M, N, K = 4, 8, 128
    X = g.standard_normal((M, K)).astype(np.float32)
    Wd = g.standard_normal((K, N)).astype(np.float32)
    A = np.concatenate([orc.pack_q8_1(r) for r in X])
    Bq = orc.legacy_pack_q4k_col(Wd, K, N)
    got = orc.legacy_qmm(A, Bq, M, N, K)
    qa, da, _ = _q8_fields(A)
    xa = (qa * da[:, None]).reshape(M, K)
    bb = Bq.reshape(N, K // 32, 20)
    d4 = bb[:, :, 16:18].copy().view(np.float16).astype(np.float64)[..., 0]
    dm = bb[:, :, 18:20].copy().view(np.float16).astype(np.float64)[..., 0]
    nib = np.empty((N, K // 32, 32))
    nib[:, :, 0::2] = bb[:, :, :16] & 15
    nib[:, :, 1::2] = bb[:, :, :16] >> 4
    w = (d4[..., None] * nib + dm[..., None]).reshape(N, K)
    ref = xa @ w.T
    assert np.allclose(got, ref, rtol=1e-4, atol=1e-4)
    # and the quantized product is a sane approximation of the dense one
    assert np.abs(got - X @ Wd).max() < 0.2 * np.abs(X @ Wd).max()


# ------------------------------------------------------------------ 144-byte super-block
def _block(d, dmin, sc, m, nib256):
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.array([d], np.float16).view(np.uint8)
    blk[2:4] = np.array([dmin], np.float16).view(np.uint8)
    return blk, sc, m, nib256


def test_q4k_scales_hand_packed(orc):
    # Hand-packed per the ggml layout: sc = 1,2,3,4,33,34,35,36 ; m = 5,6,7,8,49,50,51,52
    # j<4 : scales[j]   = sc[j]   | (sc[j+4]>>4)<<6 -> 33>>4 = 2 -> 0x80 | sc
    #       scales[j+4] = m[j]    | (m[j+4]>>4)<<6  -> 49>>4 = 3 -> 0xC0 | m
    #       scales[j+8] = (sc[j+4]&15) | (m[j+4]&15)<<4
    raw = np.array([0x81, 0x82, 0x83, 0x84, 0xC5, 0xC6, 0xC7, 0xC8, 0x11, 0x22, 0x33, 0x44], np.uint8)
    sc, m = orc.q4k_unpack_scales(raw)
    assert sc.tolist() == [1, 2, 3, 4, 33, 34, 35, 36]
    assert m.tolist() == [5, 6, 7, 8, 49, 50, 51, 52]
    assert np.array_equal(orc.q4k_pack_scales(sc, m), raw)
    assert np.array_equal(synth.pack_q4k_scales(sc, m), raw)


def test_q4k_scales_round_trip_random(orc):
    g = synth.rng(7)
    for _ in range(2000):
        raw = g.integers(0, 256, 12, dtype=np.uint8)
        sc, m = orc.q4k_unpack_scales(raw)
        assert sc.max() < 64 and m.max() < 64
        assert np.array_equal(orc.q4k_pack_scales(sc, m), raw)
    sc = g.integers(0, 64, (500, 8), dtype=np.uint8); m = g.integers(0, 64, (500, 8), dtype=np.uint8)
    packed = synth.pack_q4k_scales(sc, m)
    for i in range(500):
        s2, m2 = orc.q4k_unpack_scales(packed[i])
        assert np.array_equal(s2, sc[i]) and np.array_equal(m2, m[i])


def test_q4k_dequant_hand_block(orc):
    # d = 1, dmin = 0.5, sc_j = j+1, m_j = 2j ; qs byte i = (i & 15) | ((15 - (i & 15)) << 4)
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.array([1.0], np.float16).view(np.uint8)
    blk[2:4] = np.array([0.5], np.float16).view(np.uint8)
    sc = np.arange(1, 9, dtype=np.uint8); m = (2 * np.arange(8)).astype(np.uint8)
    blk[4:16] = synth.pack_q4k_scales(sc, m)
    i = np.arange(128)
    blk[16:] = (i & 15) | ((15 - (i & 15)) << 4)
    w = orc.q4k_dequant(blk)
    nib = orc.q4k_nibbles(blk)
    # spot values worked out by hand from the layout:
    # e=0   : group 0 low  nibble of qs[0]  = 0 , sub-block 0: 1*1*0  - 0.5*0  = 0
    # e=5   : low nibble of qs[5] = 5       , sub-block 0: 1*5      - 0      = 5
    # e=37  : high nibble of qs[5] = 10     , sub-block 1: 2*10     - 0.5*2  = 19
    # e=64  : low nibble of qs[32] = 0      , sub-block 2: 3*0      - 0.5*4  = -2
    # e=100 : group 1 high, l=4: qs[36] hi = 11 , sub-block 3: 4*11 - 0.5*6  = 41
    # e=255 : group 3 high, l=31: qs[127] hi = 0, sub-block 7: 8*0  - 0.5*14 = -7
    # e=200 : group 3 low, l=8: qs[104] lo = 8 , sub-block 6: 7*8   - 0.5*12 = 50
    for e, nv, wv in [(0, 0, 0.0), (5, 5, 5.0), (37, 10, 19.0), (64, 0, -2.0), (100, 11, 41.0),
                      (255, 0, -7.0), (200, 8, 50.0)]:
        assert nib[e] == nv, e
        assert w[e] == wv, e


def _decode_q4k_numpy(W, N, K):
    """Independent numpy decode used only to cross-check whole matrices."""
    b = W.reshape(N, K // 256, 144)
    d = b[..., 0:2].copy().view(np.float16).astype(np.float64)[..., 0]
    dmin = b[..., 2:4].copy().view(np.float16).astype(np.float64)[..., 0]
    s = b[..., 4:16].astype(np.int64)
    sc = np.empty(b.shape[:2] + (8,), np.int64); m = np.empty_like(sc)
    sc[..., :4] = s[..., 0:4] & 63
    m[..., :4] = s[..., 4:8] & 63
    sc[..., 4:] = (s[..., 8:12] & 15) | ((s[..., 0:4] >> 6) << 4)
    m[..., 4:] = (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)
    qs = b[..., 16:].reshape(N, K // 256, 4, 32).astype(np.int64)
    nib = np.stack([qs & 15, qs >> 4], axis=3)             # [N, nb, 4, 2, 32] -> sub-block j = 2g+h
    nib = nib.reshape(N, K // 256, 8, 32)
    return d, dmin, sc, m, nib


def test_q4k_gemv_f32_vs_numpy_and_integer_case(orc):
    g = synth.rng(8)
    N, K = 64, 1024
    W = synth.q4k_random(g, N, K)
    x = g.standard_normal(K).astype(np.float32)
    d, dmin, sc, m, nib = _decode_q4k_numpy(W, N, K)
    w = (d[..., None, None] * sc[..., None] * nib - (dmin[..., None] * m)[..., None]).reshape(N, K)
    wf = orc.q4k_dequant(W).reshape(N, K)
    assert np.allclose(wf, w, rtol=1e-6, atol=1e-9)
    assert np.array_equal(orc.q4k_nibbles(W).reshape(N, K // 256, 8, 32), nib)
    ref = w @ x.astype(np.float64)
    y64 = orc.gemv_q4k_f32(W, x, N, K, acc64=True)
    y32 = orc.gemv_q4k_f32(W, x, N, K, acc64=False)
    scale = np.sqrt(np.mean(ref ** 2))
    assert np.abs(y64 - ref).max() <= 2e-6 * scale
    assert np.abs(y32 - ref).max() <= 1e-4 * scale
    # d=1, dmin=0, every scale 1 and integer x: the GEMV is an exact integer dot of the nibbles
    Wi = W.copy()
    Wi[:, 0:2] = np.array([1.0], np.float16).view(np.uint8)
    Wi[:, 2:4] = 0
    Wi[:, 4:16] = synth.pack_q4k_scales(np.ones(8, np.uint8), np.zeros(8, np.uint8))
    xi = g.integers(-7, 8, K).astype(np.float32)
    yi = orc.gemv_q4k_f32(Wi, xi, N, K, acc64=False)
    assert np.array_equal(yi, (nib.reshape(N, K) @ xi.astype(np.int64)).astype(np.float32))


def test_q4k_q8_1_subdots_and_gemv(orc):
    g = synth.rng(9)
    N, K = 48, 2048
    W = synth.q4k_random(g, N, K)
    x = g.standard_normal(K).astype(np.float32)
    xq = orc.pack_q8_1(x)
    q8, d8, s8 = _q8_fields(xq)
    d, dmin, sc, m, nib = _decode_q4k_numpy(W, N, K)
    I_ref = np.einsum("nbjl,bjl->nbj", nib, q8.reshape(K // 256, 8, 32).astype(np.int64)).reshape(N, K // 32)
    I = orc.q4k_q8_1_subdots(W, xq, N, K)
    assert I.dtype == np.int32 and np.array_equal(I, I_ref)
    d8b = d8.reshape(K // 256, 8); s8b = s8.reshape(K // 256, 8)
    ref = (d[..., None] * sc * d8b * I_ref.reshape(N, K // 256, 8)).sum((1, 2)) - (dmin[..., None] * m * s8b).sum((1, 2))
    y64 = orc.gemv_q4k_q8_1(W, xq, N, K, acc64=True)
    y32 = orc.gemv_q4k_q8_1(W, xq, N, K, acc64=False)
    scale = np.sqrt(np.mean(ref ** 2))
    assert np.abs(y64 - ref).max() <= 2e-6 * scale
    assert np.abs(y32 - ref).max() <= 1e-4 * scale
    # the Q8_1 product approximates the unquantized-activation product
    yf = orc.gemv_q4k_f32(W, x, N, K)
    assert np.abs(y64 - yf).max() < 0.05 * scale + 0.05 * np.abs(yf).max()
    # sign of the min term: raising every min by one lowers y by dmin * sum(s8) per block
    W2 = W.copy().reshape(-1, 144)
    dd, dm2, sc2, m2, _ = _decode_q4k_numpy(W2, N, K)
    ok = (m2.reshape(-1, 8).max(1) < 63)
    m3 = m2.reshape(-1, 8).copy(); m3[ok] += 1
    W2[:, 4:16] = synth.pack_q4k_scales(sc2.reshape(-1, 8), m3)
    y2 = orc.gemv_q4k_q8_1(W2, xq, N, K, acc64=True)
    delta = -(dm2 * ok.reshape(N, -1) * s8b.sum(1)).sum(1)
    assert np.allclose(y2 - y64, delta, rtol=1e-3, atol=1e-5 * scale)


def test_q4k_from_dense_reconstructs(orc):
    g = synth.rng(10)
    w = (g.standard_normal((16, 512)) * 0.05).astype(np.float32)
    q = synth.q4k_from_dense(w)
    back = orc.q4k_dequant(q).reshape(16, 512)
    err = np.abs(back - w).max()
    assert err < 0.05 * 0.25, err                           # 4-bit steps over a ~6 sigma range
