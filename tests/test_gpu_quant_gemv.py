"""GPU parity, through the C ABI, of the Q8_1 quantizer, the nibble dequant kernels and the
Q4_K GEMVs against the CPU oracle on the same seeded inputs.

Bars: integer / byte outputs bit-exact; f32 outputs |gpu - ref| <= 1e-4 * max(|ref|, rms(ref))."""
import numpy as np
import pytest

from bunker_amd import runtime as rt
from bunker_amd import synth

pytestmark = pytest.mark.gpu

REL = 1e-4


def _assert_rel(got, ref, rel=REL):
    ref = ref.astype(np.float64); got = got.astype(np.float64)
    lim = rel * np.maximum(np.abs(ref), np.sqrt(np.mean(ref * ref)))
    bad = np.abs(got - ref) > lim
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside tolerance, worst {np.abs(got - ref).max():.3e}"


class Dev:
    """Uploads arrays and frees them at the end of a test."""

    def __init__(self):
        self.ptrs = []

    def up(self, a):
        p = rt.to_device(a); self.ptrs.append(p); return p

    def empty(self, nbytes):
        p = rt.cuAlloc(nbytes); self.ptrs.append(p); return p

    def close(self):
        for p in self.ptrs:
            rt.cuFree(p)


@pytest.fixture()
def dev():
    d = Dev()
    yield d
    d.close()


# ------------------------------------------------------------------ quantizer
@pytest.mark.parametrize("K,batch", [(2048, 1), (6144, 1), (2048, 8), (256, 3), (40, 2)])
def test_quantize_q8_1_bit_exact(orc, dev, K, batch):
    print(f"quantize K={K} batch={batch}", flush=True)
    g = synth.rng(100 + K + batch)
    x = g.standard_normal((batch, K)).astype(np.float32)
    x[0, :32] = 0.0
    if K >= 64:
        x[0, 32] = 127.0
        x[0, 33:41] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.49999997, -0.50000006]
        x[0, 41:64] = 0
    nb = (K + 31) // 32
    out = dev.empty(batch * nb * 36)
    rt.quantize_q8_1(dev.up(x), out, K, batch, rt.F32)
    got = rt.from_device(out, (batch, nb * 36), np.uint8)
    ref = np.stack([orc.pack_q8_1(r) for r in x])
    assert np.array_equal(got, ref)
    # bf16 activations are widened first
    xb = synth.f32_to_bf16(x)
    rt.quantize_q8_1(dev.up(xb), out, K, batch, rt.BF16)
    got = rt.from_device(out, (batch, nb * 36), np.uint8)
    ref = np.stack([orc.pack_q8_1(r) for r in synth.bf16_to_f32(xb)])
    assert np.array_equal(got, ref)


def test_quantize_q8_1_scale_sweep(orc, dev):
    """Magnitudes from 1e-6 to 1e4 and exact .5 quotients: rounding and fp16 truncation paths."""
    g = synth.rng(7)
    K = 32 * 512
    x = (g.standard_normal(K) * 10.0 ** g.uniform(-6, 4, K // 32).repeat(32)).astype(np.float32)
    half = (g.integers(-254, 254, K // 2) * 0.5).astype(np.float32)       # amax 127 -> d = 1
    half[::32] = 127.0
    x[: K // 2] = half
    out = dev.empty(K // 32 * 36)
    rt.quantize_q8_1(dev.up(x), out, K, 1, rt.F32)
    assert np.array_equal(rt.from_device(out, (K // 32 * 36,), np.uint8), orc.pack_q8_1(x))


# ------------------------------------------------------------------ dequant
def test_dequant_legacy_known_answer(orc, dev):
    g = synth.rng(8)
    nb = 128 * 32                                            # tests/test_dequant.ts:3-7 sizes
    lo = g.integers(0, 16, (nb, 16)); hi = g.integers(0, 16, (nb, 16))
    blocks = np.zeros((nb, 20), np.uint8)
    blocks[:, :16] = lo | (hi << 4)
    blocks[:, 16:] = g.integers(0, 256, (nb, 4))
    ref = np.empty((nb, 32), np.int8); ref[:, 0::2] = lo - 8; ref[:, 1::2] = hi - 8
    out = dev.empty(nb * 32)
    rt.dequant_legacy_i8(dev.up(blocks), out, nb)
    got = rt.from_device(out, (nb, 32), np.int8)
    assert np.array_equal(got, ref)
    assert np.array_equal(got.ravel(), orc.legacy_dequant_i8(blocks))


def test_q4k_unpack_bit_exact(orc, dev):
    g = synth.rng(9)
    N, K = 96, 2048
    W = synth.q4k_random(g, N, K)
    nblk = N * K // 256
    dW = dev.up(W)
    o1 = dev.empty(nblk * 256)
    rt.q4k_nibbles(dW, o1, nblk)
    assert np.array_equal(rt.from_device(o1, (nblk * 256,), np.uint8), orc.q4k_nibbles(W))
    o2 = dev.empty(nblk * 256 * 4)
    rt.q4k_dequant_f32(dW, o2, nblk)
    assert np.array_equal(rt.from_device(o2, (nblk * 256,), np.float32).view(np.uint32),
                          orc.q4k_dequant(W).view(np.uint32))


# ------------------------------------------------------------------ GEMV
DECODE_SHAPES = {"qkv": (6144, 2048), "gate_up": (12288, 2048), "down": (2048, 6144), "lm_head": (151936, 2048)}


@pytest.mark.parametrize("name", list(DECODE_SHAPES))
def test_gemv_q4k_q8_1_decode_shapes(orc, dev, name):
    N, K = DECODE_SHAPES[name]
    print(f"gemv {name} N={N} K={K}", flush=True)
    g = synth.rng(200 + N % 97)
    W = synth.q4k_random(g, N, K)
    x = g.standard_normal(K).astype(np.float32)
    dW, dx = dev.up(W), dev.up(x)
    dxq = dev.empty(K // 32 * 36)
    rt.quantize_q8_1(dx, dxq, K, 1, rt.F32)
    xq = rt.from_device(dxq, (K // 32 * 36,), np.uint8)
    assert np.array_equal(xq, orc.pack_q8_1(x))
    # exact integer sub-block dots
    dI = dev.empty(N * (K // 32) * 4)
    rt.q4k_q8_1_subdots(dW, dxq, dI, N, K)
    I = rt.from_device(dI, (N, K // 32), np.int32)
    assert np.array_equal(I, orc.q4k_q8_1_subdots(W, xq, N, K))
    # f32 output
    dy = dev.empty(N * 4)
    rt.gemv_q4k_q8_1(dW, dxq, dy, N, K)
    y = rt.from_device(dy, (N,), np.float32)
    ref = orc.gemv_q4k_q8_1(W, xq, N, K, acc64=True)
    _assert_rel(y, ref)
    # every term after the integer dots is exact in double, so the f32 result equals the host's to the bit
    assert np.array_equal(y.view(np.uint32), ref.view(np.uint32)), int((y != ref).sum())
    # run-to-run determinism (fixed reduction order, no atomics)
    rt.gemv_q4k_q8_1(dW, dxq, dy, N, K)
    assert np.array_equal(rt.from_device(dy, (N,), np.float32).view(np.uint32), y.view(np.uint32))


@pytest.mark.parametrize("N,K", [(1001, 2048), (515, 4096), (258, 6144)])
def test_gemv_variants_return_the_same_bits(orc, dev, N, K):
    """Every kernel variant behind bk_gemv_q4k_q8_1 (rows through LDS; direct loads with 1, 2 or 4 rows per wave step;
    few or many workgroups per CU) returns the checker's bits: the arithmetic does not depend on the launch shape."""
    print(f"gemv variants N={N} K={K}", flush=True)
    g = synth.rng(350 + N)
    W = synth.q4k_random(g, N, K)
    xq = orc.pack_q8_1(g.standard_normal(K).astype(np.float32))
    ref = orc.gemv_q4k_q8_1(W, xq, N, K)
    dW, dxq, dy = dev.up(W), dev.up(xq), dev.empty(N * 4)
    try:
        for impl, rpi, cap in [(2, 0, 16), (2, 4, 16), (2, 2, 1), (0, 1, 16), (0, 2, 2), (0, 4, 1), (0, 4, 64)]:
            rt.tune_set("gemv_impl", impl); rt.tune_set("gemv_rpi", rpi); rt.tune_set("gemv_cap", cap)
            rt.cuMemset(dy, 0xCD, N * 4)
            rt.gemv_q4k_q8_1(dW, dxq, dy, N, K)
            y = rt.from_device(dy, (N,), np.float32)
            assert np.array_equal(y.view(np.uint32), ref.view(np.uint32)), (impl, rpi, cap, int((y != ref).sum()))
    finally:
        rt.tune_set("gemv_impl", 2); rt.tune_set("gemv_rpi", 0); rt.tune_set("gemv_cap", 16)


@pytest.mark.parametrize("N,K", [(64, 256), (33, 768), (100, 1792), (128, 4096), (77, 8192), (5, 2048)])
def test_gemv_q4k_q8_1_ragged_shapes(orc, dev, N, K):
    print(f"gemv ragged N={N} K={K}", flush=True)
    g = synth.rng(300 + N + K)
    W = synth.q4k_random(g, N, K)
    xq = orc.pack_q8_1(g.standard_normal(K).astype(np.float32))
    dW, dxq = dev.up(W), dev.up(xq)
    dy = dev.empty(N * 4)
    rt.gemv_q4k_q8_1(dW, dxq, dy, N, K)
    y = rt.from_device(dy, (N,), np.float32); ref = orc.gemv_q4k_q8_1(W, xq, N, K)
    _assert_rel(y, ref)
    assert np.array_equal(y.view(np.uint32), ref.view(np.uint32))
    dI = dev.empty(N * (K // 32) * 4)
    rt.q4k_q8_1_subdots(dW, dxq, dI, N, K)
    assert np.array_equal(rt.from_device(dI, (N, K // 32), np.int32), orc.q4k_q8_1_subdots(W, xq, N, K))


def test_gemv_q4k_q8_1_epilogues_and_batch(orc, dev):
    g = synth.rng(11)
    N, K, B = 2048, 2048, 3
    W = synth.q4k_random(g, N, K)
    x = g.standard_normal((B, K)).astype(np.float32)
    xq = np.stack([orc.pack_q8_1(r) for r in x])
    res = synth.f32_to_bf16(g.standard_normal((B, N)).astype(np.float32))
    dW, dxq, dres = dev.up(W), dev.up(xq), dev.up(res)
    ref = np.stack([orc.gemv_q4k_q8_1(W, xq[b], N, K) for b in range(B)])
    dy = dev.empty(B * N * 4)
    rt.gemv_q4k_q8_1(dW, dxq, dy, N, K, batch=B)
    y = rt.from_device(dy, (B, N), np.float32)
    _assert_rel(y, ref)
    assert np.array_equal(y.view(np.uint32), ref.view(np.uint32))
    # bf16 output: exactly the RNE rounding of the kernel's own f32 result
    rt.gemv_q4k_q8_1(dW, dxq, dy, N, K, batch=B, out_dtype=rt.BF16)
    yb = rt.from_device(dy, (B, N), np.uint16)
    assert np.array_equal(yb, synth.f32_to_bf16(y))
    # cast then add: bf16(f32(bf16(acc)) + f32(res))  (src/model.ts:110-117 order)
    rt.gemv_q4k_q8_1(dW, dxq, dy, N, K, batch=B, out_dtype=rt.BF16, residual=dres)
    ya = rt.from_device(dy, (B, N), np.uint16)
    assert np.array_equal(ya, orc.add_bf16(yb.ravel(), res.ravel()).reshape(B, N))


def test_gemv_q4k_f32_config1(orc, dev):
    """BASELINE configs[0]: W 4096x4096, d,dmin = |N(0,0.01)|, scales/mins 0..63, nibbles 0..15, x ~ N(0,1)."""
    g = synth.rng(12)
    N = K = 4096
    W = synth.q4k_random(g, N, K)
    x = g.standard_normal(K).astype(np.float32)
    dy = dev.empty(N * 4)
    rt.gemv_q4k_f32(dev.up(W), dev.up(x), dy, N, K)
    _assert_rel(rt.from_device(dy, (N,), np.float32), orc.gemv_q4k_f32(W, x, N, K, acc64=True))


@pytest.mark.parametrize("N,K", [(64, 2048), (50, 1024), (9, 6144)])
def test_gemv_q4k_f32_other_shapes(orc, dev, N, K):
    g = synth.rng(13 + K)
    W = synth.q4k_random(g, N, K)
    x = g.standard_normal(K).astype(np.float32)
    dy = dev.empty(N * 4)
    rt.gemv_q4k_f32(dev.up(W), dev.up(x), dy, N, K)
    _assert_rel(rt.from_device(dy, (N,), np.float32), orc.gemv_q4k_f32(W, x, N, K, acc64=True))


def test_gemv_integer_special_case_exact(orc, dev):
    """d = 1, dmin = 0, scales 1, x integers with d8 = 1: the GEMV is an exact integer dot."""
    g = synth.rng(14)
    N, K = 256, 2048
    W = synth.q4k_random(g, N, K)
    W[:, 0:2] = np.array([1.0], np.float16).view(np.uint8); W[:, 2:4] = 0
    W[:, 4:16] = synth.pack_q4k_scales(np.ones(8, np.uint8), np.zeros(8, np.uint8))
    x = g.integers(-100, 101, K).astype(np.float32)
    x[::32] = 127.0                                          # every block: amax 127 -> d8 = 1
    xq = orc.pack_q8_1(x)
    dy = dev.empty(N * 4)
    rt.gemv_q4k_q8_1(dev.up(W), dev.up(xq), dy, N, K)
    nib = orc.q4k_nibbles(W).reshape(N, K).astype(np.int64)
    assert np.array_equal(rt.from_device(dy, (N,), np.float32), (nib @ x.astype(np.int64)).astype(np.float32))


def test_gemm_op_launch_surface(orc, dev):
    """The graph's gemm node through compileAndLoad + cuLaunch: A bf16 -> Q8_1 -> GEMV, slots (A, B, out)."""
    g = synth.rng(15)
    N, K = 6144, 2048
    W = synth.q4k_random(g, N, K)
    a = synth.f32_to_bf16(g.standard_normal(K).astype(np.float32))
    k = rt.compileAndLoad(f"gemm N={N} K={K} cast=1")
    dout = dev.empty(N * 2)
    rc = rt.cuLaunch(k, [1, N // 64, 1], [128, 1, 1], [dev.up(a), dev.up(W), dout])
    assert rc == 0, rt.last_error()
    rt.cuSync()
    xq = orc.pack_q8_1(synth.bf16_to_f32(a))
    ref = orc.gemv_q4k_q8_1(W, xq, N, K)
    got = synth.bf16_to_f32(rt.from_device(dout, (N,), np.uint16))
    assert np.all(np.abs(got - ref) <= 2.0 ** -8 * np.abs(ref) + 1e-4 * np.sqrt(np.mean(ref ** 2)))
    # error paths: too few slots, unknown op, bad K
    assert rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], [0, 0]) < 0 and "slots" in rt.last_error()
    with pytest.raises(rt.BunkerError, match="no kernel for op"):
        rt.compileAndLoad("nonsense N=1")
    with pytest.raises(rt.BunkerError, match="multiple of 256"):
        rt.compileAndLoad("gemm N=16 K=100")
    with pytest.raises(rt.BunkerError, match="multiple of 256"):
        rt.gemv_q4k_q8_1(1 << 20, 1 << 20, 1 << 20, 16, 100)


@pytest.mark.parametrize("N,K,B", [(6144, 2048, 32), (2048, 6144, 32), (16, 2048, 32), (100, 768, 7), (2048, 4096, 17),
                                   (4096, 2048, 40), (520, 512, 100)])
def test_gemm_mfma_equals_gemv_and_oracle(orc, dev, N, K, B):
    """Batched int8-MFMA matmul: same bits as the GEMV path and as the host loop in double, for every batch row."""
    print(f"gemm mfma N={N} K={K} B={B}", flush=True)
    g = synth.rng(700 + N + K + B)
    W = synth.q4k_random(g, N, K)
    x = g.standard_normal((B, K)).astype(np.float32)
    x[0] = 0.0                                              # an all-zero activation row
    xq = np.stack([orc.pack_q8_1(r) for r in x])
    res = synth.f32_to_bf16(g.standard_normal((B, N)).astype(np.float32))
    dW, dxq, dres = dev.up(W), dev.up(xq), dev.up(res)
    dy, dy2 = dev.empty(B * N * 4), dev.empty(B * N * 4)
    rt.gemm_q4k_q8_1(dW, dxq, dy, N, K, B)
    y = rt.from_device(dy, (B, N), np.float32)
    ref = np.stack([orc.gemv_q4k_q8_1(W, xq[b], N, K) for b in range(B)])
    _assert_rel(y, ref)
    assert np.array_equal(y.view(np.uint32), ref.view(np.uint32)), int((y != ref).sum())
    rt.gemv_q4k_q8_1(dW, dxq, dy2, N, K, batch=B)
    assert np.array_equal(rt.from_device(dy2, (B, N), np.float32).view(np.uint32), y.view(np.uint32))
    rt.gemm_q4k_q8_1(dW, dxq, dy, N, K, B, out_dtype=rt.BF16, residual=dres)
    ya = rt.from_device(dy, (B, N), np.uint16)
    assert np.array_equal(ya, orc.add_bf16(synth.f32_to_bf16(y).ravel(), res.ravel()).reshape(B, N))


@pytest.mark.parametrize("N,K,B", [(200, 2048, 70), (96, 1280, 32), (41, 3072, 19)])
def test_gemm_mfma_every_split_of_k_returns_the_same_bits(orc, dev, N, K, B):
    """1, 2, 4 or 8 wavefronts per tile (K split by super-block, partials joined in wave order): same bits as the host loop."""
    print(f"gemm mfma splits N={N} K={K} B={B}", flush=True)
    g = synth.rng(900 + N + K + B)
    W = synth.q4k_random(g, N, K)
    x = (g.standard_normal((B, K)) * np.exp(g.standard_normal((B, 1)))).astype(np.float32)
    xq = np.stack([orc.pack_q8_1(r) for r in x])
    ref = np.stack([orc.gemv_q4k_q8_1(W, xq[b], N, K) for b in range(B)])
    dW, dxq, dy = dev.up(W), dev.up(xq), dev.empty(B * N * 4)
    try:
        for r16 in (0, 1, 2):                  # tiles of 32, 16 or 8 weight rows (the narrow ones for a single batch tile only)
            rt.tune_set("gemm_r16", r16)
            for nw in (1, 2, 4, 8):
                rt.tune_set("gemm_nw", nw)
                rt.cuMemset(dy, 0xff, B * N * 4)
                rt.gemm_q4k_q8_1(dW, dxq, dy, N, K, B)
                y = rt.from_device(dy, (B, N), np.float32)
                assert np.array_equal(y.view(np.uint32), ref.view(np.uint32)), (r16, nw, int((y != ref).sum()))
    finally:
        rt.tune_set("gemm_nw", 0)
        rt.tune_set("gemm_r16", -1)
