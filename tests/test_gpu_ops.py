"""GPU parity of the glue ops, the gated-DeltaNet step and the paged decode attention against
the CPU oracle.  The glue ops and the fused GDN / attention ops go through the reference's
launch surface (compileAndLoad + cuLaunch with 8-byte slots in model.ts's argument order);
the core GDN recurrence and the paged attention also through their typed C entry points.

Bars: bf16 outputs within 2e-2 max-abs and f32 state / lse within 1e-4 relative where the
arithmetic leaves freedom (attention, the core GDN entry point); everything else is bit-exact,
because kernels and checker share the arithmetic rules (reductions and transcendentals in
double, rounded once; no implicit fused multiply-add)."""
import numpy as np
import pytest

from bunker_amd import runtime as rt
from bunker_amd import synth

pytestmark = pytest.mark.gpu

bf = synth.f32_to_bf16
f32 = synth.bf16_to_f32
G3 = [1, 1, 1]
B128 = [128, 1, 1]


class Dev:
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


def launch(spec, args):
    k = rt.compileAndLoad(spec)
    rc = rt.cuLaunch(k, G3, B128, args)
    assert rc == 0, rt.last_error()
    rt.cuSync()


def bf16_close(got_bits, ref_bits, ulps=1.0, atol=1e-6):
    """bf16 results equal up to `ulps` bf16 roundings of the reference magnitude."""
    g = f32(got_bits).astype(np.float64); r = f32(ref_bits).astype(np.float64)
    lim = ulps * 2.0 ** -8 * np.abs(r) + atol
    bad = np.abs(g - r) > lim
    assert not bad.any(), f"{bad.sum()} of {bad.size} differ, worst {np.abs(g - r).max():.3e}"
    assert np.abs(g - r).max() <= 2e-2 * max(1.0, np.abs(r).max())


# ------------------------------------------------------------------ glue
@pytest.mark.parametrize("N", [32, 1024, 2016, 2048, 2080, 4096, 6144])
def test_rmsnorm_row_lengths(orc, dev, N):
    """Rows that fit a workgroup's registers (up to 2048 elements, also with idle threads) and rows that take the loop."""
    print(f"rmsnorm N={N}", flush=True)
    g = synth.rng(430 + N)
    rows = 3
    x = bf((g.standard_normal((rows, N)) * np.exp(g.standard_normal((rows, 1)))).astype(np.float32))
    w = bf((g.standard_normal(N) * 0.1).astype(np.float32))
    ref = np.stack([orc.rmsnorm(r, w) for r in x])
    dx, dw, dn, dxq = dev.up(x), dev.up(w), dev.empty(rows * N * 2), dev.empty(rows * N // 32 * 36)
    launch(f"rmsnorm N={N} batch={rows}", [dx, dw, dn])
    assert np.array_equal(rt.from_device(dn, (rows, N), np.uint16), ref)
    rt.cuMemset(dn, 0xff, rows * N * 2)
    launch(f"rmsnorm_q8_1 N={N} batch={rows}", [dx, dw, dn, dxq])
    assert np.array_equal(rt.from_device(dn, (rows, N), np.uint16), ref)
    xq = rt.from_device(dxq, (rows, N // 32 * 36), np.uint8)
    assert np.array_equal(xq, np.stack([orc.pack_q8_1(f32(r)) for r in ref]))


@pytest.mark.parametrize("batch", [1, 4])
def test_embed_rmsnorm_cast_add_swiglu(orc, dev, batch):
    print(f"glue batch={batch}", flush=True)
    g = synth.rng(400 + batch)
    H, V, I = 2048, 1000, 6144
    E = bf(g.standard_normal((V, H)).astype(np.float32))
    ids = g.integers(0, V, batch).astype(np.int32)
    dE, dout = dev.up(E), dev.empty(batch * H * 2)
    if batch == 1:
        launch(f"embed H={H} VOCAB={V}", [dE, int(ids[0]), dout])
    else:
        launch(f"embed H={H} VOCAB={V} batch={batch} ids_dev=1", [dE, dev.up(ids), dout])
    x = rt.from_device(dout, (batch, H), np.uint16)
    assert np.array_equal(x, E[ids])
    # rmsnorm
    w = bf((g.standard_normal(H) * 0.1).astype(np.float32))
    dn = dev.empty(batch * H * 2)
    launch(f"rmsnorm N={H} batch={batch}", [dout, dev.up(w), dn])
    y = rt.from_device(dn, (batch, H), np.uint16)
    ref = np.stack([orc.rmsnorm(r, w) for r in x])
    assert np.array_equal(y, ref)
    # rmsnorm + Q8_1 in one kernel: same bf16 output, and the blocks are the quantizer's of that output
    dxq = dev.empty(batch * H // 32 * 36); dn2 = dev.empty(batch * H * 2)
    launch(f"rmsnorm_q8_1 N={H} batch={batch}", [dout, dev.up(w), dn2, dxq])
    y2 = rt.from_device(dn2, (batch, H), np.uint16)
    assert np.array_equal(y2, y)
    xq = rt.from_device(dxq, (batch, H // 32 * 36), np.uint8)
    assert np.array_equal(xq, np.stack([orc.pack_q8_1(f32(r)) for r in y]))
    # cast, add, swiglu
    a = (g.standard_normal((batch, I)) * 3).astype(np.float32); u = g.standard_normal((batch, I)).astype(np.float32)
    dc = dev.empty(batch * I * 2)
    # values that reach every branch of the conversion: ties, carries into the exponent, denormals, infinities, NaN
    sp = np.array([0x3F808000, 0x3F818000, 0x3F80FFFF, 0x7F7FFFFF, 0xFF7FFFFF, 0x00000001, 0x00008000, 0x00018000, 0x807FFFFF,
                   0x7F800000, 0xFF800000, 0x7FC00000, 0x7F800001, 0xFFA12345, 0x00000000, 0x80000000, 0x33800000, 0x477FE000],
                  np.uint32).view(np.float32)
    a[0, :sp.size] = sp
    launch(f"cast N={I} batch={batch}", [dev.up(a), dc])
    got = rt.from_device(dc, (batch, I), np.uint16)
    ref = np.array([orc.lib().orc_f32_to_bf16(float(v)) if not np.isnan(v) else 0 for v in sp], np.uint16)
    nan = np.isnan(sp)
    assert np.array_equal(got[0, :sp.size][~nan], ref[~nan])
    assert np.all((got[0, :sp.size][nan] & 0x7F80) == 0x7F80) and np.all((got[0, :sp.size][nan] & 0x007F) != 0)   # NaN stays NaN
    assert np.array_equal(got[:, sp.size:], bf(a)[:, sp.size:])
    a[0, :sp.size] = 1.0          # the checker's swiglu below is for finite inputs
    launch(f"swiglu N={I} batch={batch}", [dev.up(a), dev.up(u), dc])
    assert np.array_equal(rt.from_device(dc, (batch * I,), np.uint16), orc.swiglu(a.ravel(), u.ravel()))
    p, q = bf(a), bf(u)
    launch(f"add N={I} batch={batch}", [dev.up(p), dev.up(q), dc])
    assert np.array_equal(rt.from_device(dc, (batch * I,), np.uint16), orc.add_bf16(p.ravel(), q.ravel()))


@pytest.mark.parametrize("batch", [1, 3])
def test_conv1d_decode(orc, dev, batch):
    g = synth.rng(410 + batch)
    Cn = 6144
    x = bf(g.standard_normal((batch, Cn)).astype(np.float32))
    st = bf(g.standard_normal((batch, 3, Cn)).astype(np.float32))
    w = bf((g.standard_normal((Cn, 4)) * 0.5).astype(np.float32))
    dout, dst = dev.empty(batch * Cn * 2), dev.empty(batch * 3 * Cn * 2)
    launch(f"conv1d_decode QKVD={Cn} batch={batch}", [dev.up(x), dev.up(st), dev.up(w), dout, dst])
    out = rt.from_device(dout, (batch, Cn), np.uint16); stn = rt.from_device(dst, (batch, 3, Cn), np.uint16)
    for b in range(batch):
        ro, rs = orc.conv1d_decode(x[b], st[b], w)
        assert np.array_equal(out[b], ro)
        assert np.array_equal(stn[b], rs)


@pytest.mark.parametrize("batch", [1, 2])
def test_qknorm_rope(orc, dev, batch):
    g = synth.rng(420 + batch)
    NH, NKV, HD, HALF, MAXL = 16, 2, 256, 32, 4200
    cos_t, sin_t = orc.rope_tables(MAXL, 64, 1e7)
    dcos, dsin = dev.up(cos_t), dev.up(sin_t)
    qg = bf(g.standard_normal((batch, NH, 2, HD)).astype(np.float32))
    kk = bf(g.standard_normal((batch, NKV, HD)).astype(np.float32))
    wq = bf((g.standard_normal(HD) * 0.1).astype(np.float32)); wk = bf((g.standard_normal(HD) * 0.1).astype(np.float32))
    dq, dk = dev.empty(batch * NH * HD * 2), dev.empty(batch * NKV * HD * 2)
    launch(f"qnorm HD={HD} NH={NH} batch={batch}", [dev.up(qg), dev.up(wq), dq])
    launch(f"knorm HD={HD} NKV={NKV} batch={batch}", [dev.up(kk), dev.up(wk), dk])
    qn = rt.from_device(dq, (batch, NH * HD), np.uint16); kn = rt.from_device(dk, (batch, NKV * HD), np.uint16)
    for b in range(batch):
        assert np.array_equal(qn[b], orc.headnorm(qg[b].ravel(), wq, NH, HD, 2 * HD))
        assert np.array_equal(kn[b], orc.headnorm(kk[b].ravel(), wk, NKV, HD, HD))
    pos = [4096, 17][:batch]
    if batch == 1:
        launch(f"rope HD={HD} NH={NH} ROT_HALF={HALF} MAX_LEN={MAXL}", [dq, dcos, dsin, pos[0]])
        launch(f"ropek HD={HD} NKV={NKV} ROT_HALF={HALF} MAX_LEN={MAXL}", [dk, dcos, dsin, pos[0]])
    else:
        dpos = dev.up(np.array(pos, np.int32))
        launch(f"rope HD={HD} NH={NH} ROT_HALF={HALF} MAX_LEN={MAXL} batch={batch} pos_dev=1", [dq, dcos, dsin, dpos])
        launch(f"ropek HD={HD} NKV={NKV} ROT_HALF={HALF} MAX_LEN={MAXL} batch={batch} pos_dev=1", [dk, dcos, dsin, dpos])
    qr = rt.from_device(dq, (batch, NH * HD), np.uint16); kr = rt.from_device(dk, (batch, NKV * HD), np.uint16)
    for b in range(batch):
        assert np.array_equal(qr[b], orc.rope(qn[b], cos_t, sin_t, pos[b], NH, HD, HALF))
        assert np.array_equal(kr[b], orc.rope(kn[b], cos_t, sin_t, pos[b], NKV, HD, HALF))
    # a position outside the table is refused on the host
    k = rt.compileAndLoad(f"rope HD={HD} NH={NH} ROT_HALF={HALF} MAX_LEN={MAXL}")
    assert rt.cuLaunch(k, G3, B128, [dq, dcos, dsin, MAXL]) < 0 and "outside the table" in rt.last_error()


@pytest.mark.parametrize("batch", [1, 5])
def test_argmax(orc, dev, batch):
    # prototypes/test_argmax.ts:33-44 vector, then ties / NaN / all -inf rows
    V = 248320
    data = np.tile((np.sin(np.arange(V, dtype=np.float64)) * 10).astype(np.float32), (batch, 1))
    data[0, 123456] = 999.0
    if batch > 1:
        data[1, :] = 0.0; data[1, [70000, 4097, 200000]] = 5.0          # tie: lowest index
        data[2, :] = -np.inf                                             # nothing above -FLT_MAX: index 0
        data[3, 5] = np.nan; data[3, 99999] = 50.0                       # NaN never wins
        data[4, V - 1] = 1e30                                            # last element
    dv, di = dev.empty(batch * 4), dev.empty(batch * 4)
    launch(f"argmax VOCAB={V} batch={batch}", [dev.up(data), dv, di])
    val = rt.from_device(dv, (batch,), np.float32); idx = rt.from_device(di, (batch,), np.int32)
    for b in range(batch):
        rv, ri = orc.argmax(data[b])
        assert idx[b] == ri and val[b] == np.float32(rv), (b, idx[b], ri)
    assert idx[0] == 123456 and val[0] == 999.0
    # vocab of the synthetic model, random logits
    g = synth.rng(430)
    lg = g.standard_normal((batch, 151936)).astype(np.float32)
    launch(f"argmax VOCAB=151936 batch={batch}", [dev.up(lg), dv, di])
    assert np.array_equal(rt.from_device(di, (batch,), np.int32), lg.argmax(1).astype(np.int32))


# ------------------------------------------------------------------ GDN
def _gdn_fused_inputs(g, Hg, B):
    conv = bf(g.standard_normal((B, 3 * Hg * 128)).astype(np.float32))
    z = bf(g.standard_normal((B, Hg * 128)).astype(np.float32))
    A_log = (g.standard_normal(Hg) * 0.5).astype(np.float32)
    dt_bias = bf(g.standard_normal(Hg).astype(np.float32))
    a_p = g.standard_normal((B, Hg)).astype(np.float32); b_p = g.standard_normal((B, Hg)).astype(np.float32)
    norm_w = (1 + 0.1 * g.standard_normal(128)).astype(np.float32)
    S = (g.standard_normal((B, Hg, 128, 128)) * 0.02).astype(np.float32)
    return conv, z, A_log, dt_bias, a_p, b_p, norm_w, S


@pytest.mark.parametrize("Hg,B", [(16, 1), (16, 4), (3, 2)])
def test_gdn_delta_rule_fused(orc, dev, Hg, B):
    print(f"gdn fused Hg={Hg} B={B}", flush=True)
    g = synth.rng(500 + Hg + B)
    conv, z, A_log, dt_bias, a_p, b_p, norm_w, S = _gdn_fused_inputs(g, Hg, B)
    dout, dS = dev.empty(B * Hg * 128 * 2), dev.empty(S.nbytes)
    launch(f"gdn_delta_rule LVH={Hg} LKD=128 LVD=128 batch={B}",
           [dev.up(conv), dev.up(z), dev.up(A_log), dev.up(dt_bias), dev.up(a_p), dev.up(b_p), dev.up(norm_w), dev.up(S), dout, dS])
    out = rt.from_device(dout, (B, Hg * 128), np.uint16); Sn = rt.from_device(dS, (B, Hg, 128, 128), np.float32)
    for b in range(B):
        # canonical order of the two k-reductions (fmaf chains of 16 rows, then the 8 chains in order): to the bit
        ro, rS = orc.gdn_step(conv[b], z[b], A_log, dt_bias, a_p[b], b_p[b], norm_w, S[b], Hg, rows_per_chain=16)
        assert np.array_equal(Sn[b].view(np.uint32), rS.view(np.uint32)), int((Sn[b] != rS).sum())
        assert np.array_equal(out[b], ro), int((out[b] != ro).sum())
        # and within tolerance of the order-free double accumulation
        ro2, rS2 = orc.gdn_step(conv[b], z[b], A_log, dt_bias, a_p[b], b_p[b], norm_w, S[b], Hg, rows_per_chain=0)
        assert np.abs(Sn[b] - rS2).max() <= 1e-4 * np.abs(rS2).max()
        assert np.abs(f32(out[b]).astype(np.float64) - f32(ro2)).max() <= 2e-2


@pytest.mark.parametrize("B", [1, 8])
def test_gdn_core_config3(orc, dev, B):
    """BASELINE configs[2]: 32 heads, dk=dv=128, S ~ N(0,0.02), q,k L2-normalised bf16, g=-softplus(a), beta=sigmoid."""
    print(f"gdn core B={B}", flush=True)
    g = synth.rng(510 + B)
    Hg = 32

    def l2(x):
        return bf(x / np.sqrt((x * x).sum(-1, keepdims=True)))

    q = l2(g.standard_normal((B, Hg, 128)).astype(np.float32)); k = l2(g.standard_normal((B, Hg, 128)).astype(np.float32))
    v = bf(g.standard_normal((B, Hg, 128)).astype(np.float32))
    gl = (-np.log1p(np.exp(g.standard_normal((B, Hg))))).astype(np.float32)
    beta = (1 / (1 + np.exp(-g.standard_normal((B, Hg))))).astype(np.float32)
    S = (g.standard_normal((B, Hg, 128, 128)) * 0.02).astype(np.float32)
    dS = dev.up(S); dout = dev.empty(B * Hg * 128 * 2); dSo = dev.empty(S.nbytes)
    rt.gdn_core(dev.up(q), dev.up(k), dev.up(v), dev.up(gl), dev.up(beta), dS, dout, dSo, Hg, B)
    out = rt.from_device(dout, (B, Hg * 128), np.uint16); Sn = rt.from_device(dSo, (B, Hg, 128, 128), np.float32)
    for b in range(B):
        ro, rS = orc.gdn_core(q[b], k[b], v[b], gl[b], beta[b], S[b], Hg)
        assert np.abs(Sn[b] - rS).max() <= 1e-4 * np.abs(rS).max()
        assert np.abs(f32(out[b]).astype(np.float64) - f32(ro)).max() <= 2e-2
        bf16_close(out[b], ro, ulps=1.0, atol=1e-4)
    # in place (S_out == S_in) gives the same state
    rt.gdn_core(dev.up(q), dev.up(k), dev.up(v), dev.up(gl), dev.up(beta), dS, dout, dS, Hg, B)
    assert np.array_equal(rt.from_device(dS, S.shape, np.float32).view(np.uint32), Sn.view(np.uint32))
    # beta = 0: S' = exp(g) * S (one rounding of the product; the device exp may differ from libm by an ulp)
    rt.gdn_core(dev.up(q), dev.up(k), dev.up(v), dev.up(gl), dev.up(np.zeros_like(beta)), dev.up(S), dout, dSo, Hg, B)
    S0 = rt.from_device(dSo, S.shape, np.float32)
    ok = np.allclose(S0, S * np.exp(gl)[:, :, None, None].astype(np.float32), rtol=1e-6, atol=0)
    assert ok


# ------------------------------------------------------------------ attention
def _run_attn(dev, q, kc, vc, bt, ctx, B, L, splits=0, lse=True):
    NH, NKV, HD = 16, 2, 256
    s, ws = rt.attn_plan(B, NKV, L, splits)
    dws = dev.empty(ws) if ws else 0
    dout = dev.empty(B * NH * HD * 2); dlse = dev.empty(B * NH * 4)
    rt.attn_decode(dev.up(q), dev.up(kc), dev.up(rt.v_pages_to_device_layout(vc)), dev.up(bt), bt.shape[1], dev.up(ctx), L,
                   dout, dlse if lse else 0, B, NH, NKV, HD, 16, s, dws, ws)
    return rt.from_device(dout, (B, NH, HD), np.uint16), rt.from_device(dlse, (B, NH), np.float32), s


@pytest.mark.parametrize("B,L", [(1, 4096), (8, 4096), (1, 32768), (8, 32768)])
def test_attn_decode_config4(orc, dev, B, L):
    """BASELINE configs[3]: 16 q heads, 2 KV heads, head_dim 256, 16-token pages, lengths uniform in [L/2, L]."""
    print(f"attn B={B} L={L}", flush=True)
    g = synth.rng(600 + B + L)
    kc, vc, bt, ctx = synth.paged_kv_random(g, B, L)
    q = bf(g.standard_normal((B, 16, 256)).astype(np.float32))
    out, lse, s = _run_attn(dev, q, kc, vc, bt, ctx, B, L)
    ro, rl = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, 16, 2, 256, 16)
    assert np.abs(f32(out).astype(np.float64) - f32(ro)).max() <= 2e-2
    assert np.all(np.abs(lse - rl) <= 1e-4 * np.abs(rl))


def test_attn_decode_invariants(orc, dev):
    g = synth.rng(610)
    B, L = 4, 700
    kc, vc, bt, ctx = synth.paged_kv_random(g, B, L)
    ctx[:] = [1, 17, 700, 353]                             # one token; ragged page; full; odd
    q = bf(g.standard_normal((B, 16, 256)).astype(np.float32))
    ro, rl = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, 16, 2, 256, 16)
    outs = {}
    for splits in (1, 2, 5, 0):
        out, lse, s = _run_attn(dev, q, kc, vc, bt, ctx, B, L, splits)
        outs[splits] = (out, lse)
        assert np.abs(f32(out).astype(np.float64) - f32(ro)).max() <= 2e-2, splits
        assert np.all(np.abs(lse - rl) <= 1e-4 * np.maximum(1, np.abs(rl))), splits
    # len == 1: o = v of that token exactly, lse = its score
    assert np.array_equal(outs[1][0][0], np.repeat(vc[bt[0, 0], :, 0], 8, axis=0))
    # split count changes the merge order only: results agree to rounding
    assert np.abs(f32(outs[1][0]).astype(np.float64) - f32(outs[5][0])).max() <= 1e-2
    assert np.allclose(outs[1][1], outs[5][1], rtol=1e-5, atol=1e-5)
    # permuting the physical pages (and the block table with them) leaves the output unchanged, bit for bit
    perm = g.permutation(kc.shape[0]); inv = np.empty_like(perm); inv[perm] = np.arange(perm.size)
    out_p, lse_p, _ = _run_attn(dev, q, kc[perm], vc[perm], inv[bt].astype(np.int32), ctx, B, L, 2)
    assert np.array_equal(out_p, outs[2][0]) and np.array_equal(lse_p, outs[2][1])


def test_attn_decode_splits_follow_lengths_in_device_memory(orc, dev):
    """Lengths in device memory: relative splits (tune attn_bal = 2: every sequence cuts its own pages) and the balanced
    plan (1: the batch's workgroup slots handed out in proportion to the lengths) against the plain splits of the
    bound (0).  With every length at the bound all three cut alike (same bits, also where some splits stay empty);
    ragged lengths stay within the tolerance, whether the first page budget of the plan fits the slots or not."""
    g = synth.rng(620)
    try:
        B, L = 4, 4100                          # 257 pages: the plain form leaves splits without pages
        kc, vc, bt, ctx = synth.paged_kv_random(g, B, L)
        ctx[:] = L
        q = bf(g.standard_normal((B, 16, 256)).astype(np.float32))
        rt.tune_set("attn_bal", 0)
        out0, lse0, s0 = _run_attn(dev, q, kc, vc, bt, ctx, B, L)
        assert s0 > 1
        for mode in (1, 2, -1):
            rt.tune_set("attn_bal", mode)
            out1, lse1, s1 = _run_attn(dev, q, kc, vc, bt, ctx, B, L)
            assert s0 == s1
            assert np.array_equal(out0, out1) and np.array_equal(lse0.view(np.uint32), lse1.view(np.uint32)), mode
        # ragged: one token, one page, a page and a token, long ones; many rows; a bound far above the contexts
        for B, L, lens in ((8, 8192, [1, 16, 17, 5000, 8192, 33, 4096, 8191]),
                           (64, 1024, list(g.integers(1, 1025, 64))),
                           (2, 20000, [20000, 3]),
                           (3, 32768, [900, 2100, 1500]),
                           (1, 9000, [4700])):
            print(f"attn, lengths on the device: B={B} L={L}", flush=True)
            kc, vc, bt, ctx = synth.paged_kv_random(g, B, L)
            ctx[:] = lens
            q = bf(g.standard_normal((B, 16, 256)).astype(np.float32))
            ro, rl = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, 16, 2, 256, 16)
            rt.tune_set("attn_bal", 0)
            outp, lsep, _ = _run_attn(dev, q, kc, vc, bt, ctx, B, L)
            for mode in (1, 2, -1):
                rt.tune_set("attn_bal", mode)
                out, lse, s = _run_attn(dev, q, kc, vc, bt, ctx, B, L)
                assert s > 1
                assert np.abs(f32(out).astype(np.float64) - f32(ro)).max() <= 2e-2, mode
                assert np.all(np.abs(lse - rl) <= 1e-4 * np.maximum(1, np.abs(rl))), mode
                assert np.abs(f32(out).astype(np.float64) - f32(outp)).max() <= 1e-2, mode
                assert np.allclose(lse, lsep, rtol=1e-5, atol=1e-5), mode
    finally:
        rt.tune_set("attn_bal", -1)


@pytest.mark.parametrize("batch", [1, 3])
def test_fa2_attn_op_appends_and_attends(orc, dev, batch):
    """The graph's fa2_attn node: slots (q, k, v, qgate, kv_k_in, kv_v_in, pos, out, kv_k_new, kv_v_new)."""
    g = synth.rng(620 + batch)
    NH, NKV, HD, MAXL = 16, 2, 256, 512
    ppseq = MAXL // 16
    pos = [300, 15, 16][:batch]
    kc = bf(g.standard_normal((batch * ppseq, NKV, 16, HD)).astype(np.float32))
    vc = bf(g.standard_normal((batch * ppseq, NKV, 16, HD)).astype(np.float32))
    q = bf(g.standard_normal((batch, NH, HD)).astype(np.float32))
    k = bf(g.standard_normal((batch, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((batch, NKV, HD)).astype(np.float32))
    qgate = bf(g.standard_normal((batch, NH, 2, HD)).astype(np.float32))
    dkc, dvc = dev.up(kc), dev.up(rt.v_pages_to_device_layout(vc))
    dout = dev.empty(batch * NH * HD * 2)
    if batch == 1:
        launch(f"fa2_attn HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL}",
               [dev.up(q), dev.up(k), dev.up(v), dev.up(qgate), dkc, dvc, pos[0], dout, dkc, dvc])
    else:
        launch(f"fa2_attn HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} batch={batch} pos_dev=1",
               [dev.up(q), dev.up(k), dev.up(v), dev.up(qgate), dkc, dvc, dev.up(np.array(pos, np.int32)), dout, dkc, dvc])
    out = rt.from_device(dout, (batch, NH, HD), np.uint16)
    bt = np.arange(batch * ppseq, dtype=np.int32).reshape(batch, ppseq)
    for b in range(batch):
        orc.kv_append(k[b], v[b], kc, vc, bt[b], pos[b], NKV, HD, 16)
    ctx = np.array(pos, np.int32) + 1
    ro, _ = orc.attn_decode_paged(q, kc, vc, bt, ctx, batch, NH, NKV, HD, 16, gate=qgate.ravel()[HD:],
                                  gate_bstride=NH * 2 * HD, gate_hstride=2 * HD)
    assert np.abs(f32(out).astype(np.float64) - f32(ro)).max() <= 2e-2
    # the caches now hold the appended token
    kc_d = rt.from_device(dkc, kc.shape, np.uint16)
    vc_d = rt.from_device(dvc, (batch * ppseq, NKV, HD, 16), np.uint16).transpose(0, 1, 3, 2)
    assert np.array_equal(kc_d, kc) and np.array_equal(vc_d, vc)


def test_streams_order_work_through_events(orc, dev):
    """A second stream: work queued there runs behind an event of the first stream, results are visible after cuSync,
    and a handle that is not a stream of the library is refused."""
    n = 1 << 20
    a = np.arange(n, dtype=np.float32)
    da, db, dc = dev.up(a), dev.empty(n * 4), dev.empty(n * 4)
    st = rt.Stream()
    rt.cuDtoD(db, da, n * 4)                       # first stream: b = a
    ev = rt.Event().record()
    st.wait(ev)
    with st:
        rt.cuDtoD(dc, db, n * 4)                   # second stream, behind the event: c = b
        with st:                                   # nesting keeps the selection
            pass
        done = rt.Event().record()
    rt.streamWaitEvent(done)                       # first stream waits for the second
    rt.cuSync()
    assert np.array_equal(rt.from_device(dc, (n,), np.float32), a)
    with pytest.raises(rt.BunkerError, match="not a stream"):
        rt._check(rt.cu().bk_stream_use(12345), "bk_stream_use")
    st.destroy(); ev.destroy(); done.destroy()


def test_only_launches_are_recorded_between_capture_begin_and_end():
    """Inside a capture every call that is not a launch is refused with the library's own error and leaves the capture
    open and usable (a memset node would replay wrongly, a copy or a sync would end the capture with a runtime error);
    the graph then replays the launches recorded around the refused calls."""
    import ctypes as C
    lib = rt.cu()
    x = np.arange(64, dtype=np.float32)
    dx = rt.to_device(x); dq = rt.cuAlloc(2 * 36); rt.cuMemset(dq, 0, 72)
    host = np.zeros(72, np.uint8)
    p = C.c_uint64(0)
    k_spare = rt.compileAndLoad("gemm N=64 K=256")            # owns a workspace
    with rt.Graph() as gr:
        rt.quantize_q8_1(dx, dq, 64, 1, rt.F32)
        for rc in (lib.bk_memset(dq, 0, 72), lib.bk_sync(), lib.bk_alloc(256, C.byref(p)), lib.bk_free(dq),
                   lib.bk_dtoh(host.ctypes.data_as(C.c_void_p), dq, 72), lib.bk_graph_launch(1),
                   lib.bk_kernel_create(b"gemm N=64 K=256"), lib.bk_kernel_destroy(k_spare.fn)):
            assert rc != 0 and b"not legal between bk_capture_begin and bk_capture_end" in lib.bk_last_error()
    assert gr.node_count() == 1
    # the handle the capture refused to destroy is still alive; once destroyed its slot is reused under another number
    # and the old number is refused
    slots = (C.c_uint64 * 3)(0, 0, 0)
    rt.unloadKernel(k_spare)
    k_new = rt.compileAndLoad("gemm N=64 K=256")
    assert k_new.fn != k_spare.fn and (k_new.fn & 0xfffff) == (k_spare.fn & 0xfffff)
    assert lib.bk_launch(k_spare.fn, slots, 3) != 0 and b"destroyed" in lib.bk_last_error()
    rt.unloadKernel(k_new)
    for _ in range(2):
        rt.cuMemset(dq, 0, 72)
        gr.launch(); rt.cuSync()
        got = rt.from_device(dq, (72,), np.uint8)
        assert got[:32].view(np.int8).max() == 127 and got[36:68].view(np.int8).max() == 127
    gr.destroy()
    rt.cuFree(dx); rt.cuFree(dq)
