"""The double-precision decode attention (bk_attn_decode_exact, and exact=1 of the fa2_* ops) against the CPU checker.

Both sides carry every bf16 x bf16 product and every sum in f64 and round the quotient once to f32 (then gate, then
bf16), so the bar here is EQUAL bits of the bf16 outputs — for every split count, for lengths in device memory under
each way of cutting the pages, for a ragged last page and for a permuted page table — and the f32 log-sum-exp within
one unit in the last place (the two sides subtract different reference exponents before the logarithm)."""
import numpy as np
import pytest

from bunker_amd import runtime as rt
from bunker_amd import synth
from test_gpu_ops import Dev, dev, launch  # noqa: F401  (dev is a fixture)

pytestmark = pytest.mark.gpu

bf = synth.f32_to_bf16
f32 = synth.bf16_to_f32


def _run_exact(dev, q, kc, vc, bt, ctx, B, L, splits=0, NH=16, NKV=2, gate=None, gate_bstride=0, gate_hstride=0):
    HD = 256
    s, ws = rt.attn_plan_exact(B, NKV, L, splits)
    assert ws > 0
    dws = dev.empty(ws)
    dout = dev.empty(B * NH * HD * 2); dlse = dev.empty(B * NH * 4)
    rt.attn_decode_exact(dev.up(q), dev.up(kc), dev.up(rt.v_pages_to_device_layout(vc)), dev.up(bt), bt.shape[1], dev.up(ctx), L,
                         dout, dlse, B, NH, NKV, HD, 16, s, dws, ws, gate=dev.up(gate) if gate is not None else 0,
                         gate_bstride=gate_bstride, gate_hstride=gate_hstride)
    return rt.from_device(dout, (B, NH, HD), np.uint16), rt.from_device(dlse, (B, NH), np.float32), s


def _same(out, lse, ro, rl, what=""):
    bad = out != ro
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.size} bf16 outputs differ, worst {np.abs(f32(out).astype(np.float64) - f32(ro)).max():.3e}"
    ulp = np.spacing(np.abs(rl)).astype(np.float64)
    fin = np.isfinite(rl)
    assert np.array_equal(np.isfinite(lse), fin) and np.all(np.abs(lse[fin].astype(np.float64) - rl[fin]) <= ulp[fin]), what


@pytest.mark.parametrize("B,L", [(1, 4096), (8, 4096), (1, 32768), (8, 32768)])
def test_exact_attention_config4_bits(orc, dev, B, L):
    """BASELINE configs[3] at full size: 16 q heads, 2 KV heads, head_dim 256, 16-token pages, lengths in [L/2, L]."""
    print(f"exact attn B={B} L={L}", flush=True)
    g = synth.rng(700 + B + L)
    kc, vc, bt, ctx = synth.paged_kv_random(g, B, L)
    q = bf(g.standard_normal((B, 16, 256)).astype(np.float32))
    out, lse, s = _run_exact(dev, q, kc, vc, bt, ctx, B, L)
    ro, rl = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, 16, 2, 256, 16)
    _same(out, lse, ro, rl, f"B={B} L={L} splits={s}")


def test_exact_attention_any_split_same_bits(orc, dev):
    g = synth.rng(710)
    B, L = 4, 700
    kc, vc, bt, ctx = synth.paged_kv_random(g, B, L)
    ctx[:] = [1, 17, 700, 353]                             # one token; ragged page; full; odd
    q = bf(g.standard_normal((B, 16, 256)).astype(np.float32))
    gate = bf(g.standard_normal((B, 16, 2, 256)).astype(np.float32))
    ro, rl = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, 16, 2, 256, 16)
    for splits in (1, 2, 5, 11, 0):
        out, lse, s = _run_exact(dev, q, kc, vc, bt, ctx, B, L, splits)
        _same(out, lse, ro, rl, f"splits={splits}")
    # len == 1: o = v of that token exactly
    assert np.array_equal(out[0], np.repeat(vc[bt[0, 0], :, 0], 8, axis=0))
    # output gate (the q_proj layout of the fused op: [q | gate] per head)
    rg, rlg = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, 16, 2, 256, 16, gate=gate.ravel()[256:], gate_bstride=16 * 512,
                                    gate_hstride=512)
    for splits in (1, 3):
        out, lse, _ = _run_exact(dev, q, kc, vc, bt, ctx, B, L, splits, gate=gate.ravel()[256:], gate_bstride=16 * 512, gate_hstride=512)
        _same(out, lse, rg, rlg, f"gate, splits={splits}")
    # permuted physical pages
    perm = g.permutation(kc.shape[0]); inv = np.empty_like(perm); inv[perm] = np.arange(perm.size)
    out_p, lse_p, _ = _run_exact(dev, q, kc[perm], vc[perm], inv[bt].astype(np.int32), ctx, B, L, 2)
    _same(out_p, lse_p, ro, rl, "permuted pages")
    # what lies in the cache behind a context must not matter, not even when it is no number (bf16 NaN / Inf patterns)
    kc2, vc2 = kc.copy(), vc.copy()
    for b in range(B):
        n = int(ctx[b])
        for pg in range(n // 16, bt.shape[1]):
            lo = n - pg * 16 if pg == n // 16 else 0
            kc2[bt[b, pg], :, lo:] = 0x7FC0
            vc2[bt[b, pg], :, lo:] = 0x7F80
    out_n, lse_n, _ = _run_exact(dev, q, kc2, vc2, bt, ctx, B, L, 3)
    _same(out_n, lse_n, ro, rl, "garbage behind the context")


def test_exact_attention_other_group_sizes(orc, dev):
    """4 query heads per KV head (the reference model's 8 : 2) and one head per KV head; more than 8 is refused."""
    g = synth.rng(720)
    B, L = 2, 1000
    for NH, NKV in ((8, 2), (4, 4), (3, 1)):
        kc, vc, bt, ctx = synth.paged_kv_random(g, B, L, NKV=NKV)
        q = bf(g.standard_normal((B, NH, 256)).astype(np.float32))
        ro, rl = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, NH, NKV, 256, 16)
        out, lse, _ = _run_exact(dev, q, kc, vc, bt, ctx, B, L, 0, NH=NH, NKV=NKV)
        _same(out, lse, ro, rl, f"NH={NH} NKV={NKV}")
    with pytest.raises(rt.BunkerError, match="at most 8"):
        kc, vc, bt, ctx = synth.paged_kv_random(g, 1, 64, NKV=1)
        _run_exact(dev, bf(g.standard_normal((1, 16, 256)).astype(np.float32)), kc, vc, bt, ctx, 1, 64, 1, NH=16, NKV=1)


def test_exact_attention_lengths_in_device_memory(orc, dev):
    """Every way of cutting the pages (plain ranges of the bound, each sequence's own pages, the balanced plan) gives
    the checker's bits, also where splits stay empty or a length is 0."""
    g = synth.rng(730)
    try:
        for B, L, lens in ((8, 8192, [1, 16, 17, 5000, 8192, 33, 4096, 8191]),
                           (64, 1024, list(g.integers(1, 1025, 64))),
                           (2, 20000, [20000, 3]),
                           (3, 32768, [900, 2100, 1500]),
                           (2, 4100, [4100, 4100])):
            print(f"exact attn, lengths on the device: B={B} L={L}", flush=True)
            kc, vc, bt, ctx = synth.paged_kv_random(g, B, L)
            ctx[:] = lens
            q = bf(g.standard_normal((B, 16, 256)).astype(np.float32))
            ro, rl = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, 16, 2, 256, 16)
            for mode in (0, 1, 2, -1):
                rt.tune_set("attn_bal", mode)
                out, lse, s = _run_exact(dev, q, kc, vc, bt, ctx, B, L)
                _same(out, lse, ro, rl, f"B={B} L={L} mode={mode}")
        # an empty context: zeros and lse = -inf, the other row untouched by it
        kc, vc, bt, ctx = synth.paged_kv_random(g, 2, 256)
        ctx[:] = [0, 100]
        q = bf(g.standard_normal((2, 16, 256)).astype(np.float32))
        ro, rl = orc.attn_decode_paged(q, kc, vc, bt, np.array([1, 100], np.int32), 2, 16, 2, 256, 16)
        for splits in (1, 4):
            out, lse, _ = _run_exact(dev, q, kc, vc, bt, ctx, 2, 256, splits)
            assert not out[0].any() and np.all(np.isneginf(lse[0]))
            assert np.array_equal(out[1], ro[1])
    finally:
        rt.tune_set("attn_bal", -1)


@pytest.mark.parametrize("batch", [1, 3])
def test_fa2_attn_op_exact_bits(orc, dev, batch):
    """The graph's fa2_attn node (exact=1 is its default): cache append, then attention with the checker's bits."""
    g = synth.rng(740 + batch)
    NH, NKV, HD, MAXL = 16, 2, 256, 512
    ppseq = MAXL // 16
    pos = [300, 15, 16][:batch]
    kc = bf(g.standard_normal((batch * ppseq, NKV, 16, HD)).astype(np.float32))
    vc = bf(g.standard_normal((batch * ppseq, NKV, 16, HD)).astype(np.float32))
    q = bf(g.standard_normal((batch, NH, HD)).astype(np.float32))
    k = bf(g.standard_normal((batch, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((batch, NKV, HD)).astype(np.float32))
    qgate = bf(g.standard_normal((batch, NH, 2, HD)).astype(np.float32))
    bt = np.arange(batch * ppseq, dtype=np.int32).reshape(batch, ppseq)
    kr, vr = kc.copy(), vc.copy()
    for b in range(batch):
        orc.kv_append(k[b], v[b], kr, vr, bt[b], pos[b], NKV, HD, 16)
    ro, _ = orc.attn_decode_paged(q, kr, vr, bt, np.array(pos, np.int32) + 1, batch, NH, NKV, HD, 16, gate=qgate.ravel()[HD:],
                                  gate_bstride=NH * 2 * HD, gate_hstride=2 * HD)
    for extra, equal in (("", True), (" exact=1 splits=3", True), (" exact=0", False)):
        dkc, dvc = dev.up(kc), dev.up(rt.v_pages_to_device_layout(vc))
        dout = dev.empty(batch * NH * HD * 2)
        spec = f"fa2_attn HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL}" + extra
        if batch == 1:
            launch(spec, [dev.up(q), dev.up(k), dev.up(v), dev.up(qgate), dkc, dvc, pos[0], dout, dkc, dvc])
        else:
            launch(spec + f" batch={batch} pos_dev=1",
                   [dev.up(q), dev.up(k), dev.up(v), dev.up(qgate), dkc, dvc, dev.up(np.array(pos, np.int32)), dout, dkc, dvc])
        out = rt.from_device(dout, (batch, NH, HD), np.uint16)
        if equal:
            assert np.array_equal(out, ro), spec
        else:
            assert np.abs(f32(out).astype(np.float64) - f32(ro)).max() <= 2e-2, spec


@pytest.mark.parametrize("NH,NKV,splits", [(16, 2, 0), (16, 2, 1), (16, 2, 5), (8, 2, 3), (2, 2, 0)])
def test_folded_preparation_equals_the_separate_launch(dev, NH, NKV, splits):
    """fa2_fused with the norms, the rotation and the cache append inside the attention kernel (the default) against
    the same op with the preparation as a launch of its own (prep_fused=0): the same bits in the output, in its Q8_1
    copy and in both caches.  The positions sit on both sides of page and tile borders, at 0, at the last slot of the
    cache and behind it (no append), and differ from sequence to sequence."""
    print(f"fa2_fused folded prep NH={NH} NKV={NKV} splits={splits}", flush=True)
    g = synth.rng(4300 + NH + splits)
    HD, HALF, MAXL = 256, 32, 512
    pos = np.array([0, 15, 16, 17, 63, 64, 65, 300, 447, 448, 510, 511, 512, 600], np.int32)
    B = len(pos)
    ppseq = MAXL // 16
    half_cols = 64
    cos_t = g.uniform(-1, 1, (MAXL, half_cols // 2)).astype(np.float32); sin_t = g.uniform(-1, 1, (MAXL, half_cols // 2)).astype(np.float32)
    kc = bf(g.standard_normal((B * ppseq, NKV, 16, HD)).astype(np.float32))
    vc = bf(g.standard_normal((B * ppseq, NKV, HD, 16)).astype(np.float32))
    qgate = bf(g.standard_normal((B, NH, 2, HD)).astype(np.float32))
    k = bf(g.standard_normal((B, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((B, NKV, HD)).astype(np.float32))
    qw = bf((g.standard_normal(HD) * 0.1).astype(np.float32)); kw = bf((g.standard_normal(HD) * 0.1).astype(np.float32))
    common = [dev.up(qgate), dev.up(k), dev.up(v), dev.up(qw), dev.up(kw), dev.up(cos_t), dev.up(sin_t), dev.up(pos)]
    res = []
    for folded in (1, 0):
        dkc, dvc = dev.up(kc), dev.up(vc)
        dout = dev.empty(B * NH * HD * 2); dq8 = dev.empty(B * NH * HD // 32 * 36)
        sp = f" splits={splits}" if splits else ""
        launch(f"fa2_fused HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} ROT_HALF={HALF} batch={B} pos_dev=1 q8out=1 prep_fused={folded}{sp}",
               common + [dkc, dvc, dout, dq8])
        res.append((rt.from_device(dout, (B, NH, HD), np.uint16), rt.from_device(dq8, (B, NH * HD // 32 * 36), np.uint8),
                    rt.from_device(dkc, kc.shape, np.uint16), rt.from_device(dvc, vc.shape, np.uint16)))
    (o1, q1, k1, v1), (o0, q0, k0, v0) = res
    assert np.array_equal(k1, k0) and np.array_equal(v1, v0)
    assert not np.array_equal(k0, kc) and np.array_equal(k0[-ppseq:], kc[-ppseq:])      # appended; the last sequence (behind the cache) not
    bad = (o1 != o0).reshape(B, -1).any(axis=1)
    assert not bad.any(), f"sequences {np.nonzero(bad)[0].tolist()} differ"
    assert np.array_equal(q1, q0)
