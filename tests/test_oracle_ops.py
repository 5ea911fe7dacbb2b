"""Pins the oracle's floating-point ops (GDN step, paged decode attention, glue) with
closed forms, invariants and float64 numpy restatements of the reference's host loops."""
import numpy as np

from bunker_amd import synth

bf = synth.f32_to_bf16
f32 = synth.bf16_to_f32


def _close_bf16(got_bits, ref_f64, tol=2e-2):
    got = f32(got_bits).astype(np.float64)
    lim = tol * np.maximum(1.0, np.abs(ref_f64))
    assert np.all(np.abs(got - ref_f64) <= lim), np.abs(got - ref_f64).max()


# ------------------------------------------------------------------ glue
def test_rmsnorm_closed_form(orc):
    g = synth.rng(20)
    x = bf(g.standard_normal(2048).astype(np.float32)); w = bf((g.standard_normal(2048) * 0.02).astype(np.float32))
    xf = f32(x).astype(np.float64); wf = f32(w).astype(np.float64)
    ref = xf / np.sqrt(np.mean(xf * xf) + 1e-6) * (1 + wf)       # prototypes/rmsnorm.ts:59-68
    got = f32(orc.rmsnorm(x, w)).astype(np.float64)
    assert np.all(np.abs(got - ref) <= 2.0 ** -8 * np.abs(ref) + 1e-30)   # within one bf16 rounding
    # scale invariance: rmsnorm(2x) == rmsnorm(x) up to the eps term
    x2 = bf(f32(x) * 2)
    assert np.array_equal(orc.rmsnorm(x2, w), orc.rmsnorm(x, w))


def test_swiglu_add_cast(orc):
    g = synth.rng(21)
    a = g.standard_normal(6144).astype(np.float32) * 3; u = g.standard_normal(6144).astype(np.float32)
    ref = a.astype(np.float64) / (1 + np.exp(-a.astype(np.float64))) * u          # prototypes/swiglu.ts:33-40
    got = f32(orc.swiglu(a, u)).astype(np.float64)
    assert np.all(np.abs(got - ref) <= 2.0 ** -8 * np.abs(ref) + 1e-6)
    assert np.array_equal(orc.cast_bf16(a), bf(a))
    x = bf(a); y = bf(u)
    assert np.array_equal(orc.add_bf16(x, y), bf(f32(x) + f32(y)))
    # swiglu(0, u) = 0 ; large positive gate -> g*u
    assert f32(orc.swiglu(np.zeros(4, np.float32), np.ones(4, np.float32))).tolist() == [0, 0, 0, 0]
    assert f32(orc.swiglu(np.full(1, 40.0, np.float32), np.full(1, 2.0, np.float32)))[0] == 80.0


def test_conv1d_decode(orc):
    g = synth.rng(22)
    Cn = 6144
    x = bf(g.standard_normal(Cn).astype(np.float32))
    st = bf(g.standard_normal((3, Cn)).astype(np.float32))
    w = bf((g.standard_normal((Cn, 4)) * 0.5).astype(np.float32))
    out, stn = orc.conv1d_decode(x, st, w)
    hist = np.concatenate([f32(st), f32(x)[None]], 0).astype(np.float64)       # [4, C], oldest first
    s = (f32(w).astype(np.float64).T * hist).sum(0)                            # prototypes/conv1d.ts:53-61
    ref = s / (1 + np.exp(-s))
    got = f32(out).astype(np.float64)
    assert np.all(np.abs(got - ref) <= 2.0 ** -8 * np.abs(ref) + 1e-5)
    assert np.array_equal(stn[0], st[1]) and np.array_equal(stn[1], st[2]) and np.array_equal(stn[2], x)


def test_headnorm_and_rope(orc):
    g = synth.rng(23)
    NH, HD = 16, 256
    qg = bf(g.standard_normal(NH * 2 * HD).astype(np.float32))                  # [q(256) | gate(256)] per head
    w = bf((g.standard_normal(HD) * 0.02).astype(np.float32))
    got = f32(orc.headnorm(qg, w, NH, HD, 2 * HD)).astype(np.float64).reshape(NH, HD)
    xq = f32(qg).astype(np.float64).reshape(NH, 2, HD)[:, 0]
    ref = xq / np.sqrt((xq * xq).mean(1, keepdims=True) + 1e-6) * (1 + f32(w).astype(np.float64))
    assert np.all(np.abs(got - ref) <= 2.0 ** -8 * np.abs(ref) + 1e-30)
    # rope: pos 0 is the identity; other positions are a rotation of pairs (i, i+32), dims >= 64 untouched
    cos_t, sin_t = orc.rope_tables(64, 64, 1e7)
    assert np.all(cos_t[0] == 1) and np.all(sin_t[0] == 0)
    i = np.arange(32)
    fr = 1e7 ** (-2.0 * i / 64)
    assert np.allclose(cos_t[37], np.cos(37 * fr), atol=1e-7) and np.allclose(sin_t[37], np.sin(37 * fr), atol=1e-7)
    q = bf(g.standard_normal(NH * HD).astype(np.float32))
    assert np.array_equal(orc.rope(q, cos_t, sin_t, 0, NH, HD), q)
    r = f32(orc.rope(q, cos_t, sin_t, 37, NH, HD)).astype(np.float64).reshape(NH, HD)
    qf = f32(q).astype(np.float64).reshape(NH, HD)
    z = (qf[:, :32] + 1j * qf[:, 32:64]) * np.exp(1j * 37 * fr)
    assert np.allclose(r[:, :32], z.real, atol=2e-2) and np.allclose(r[:, 32:64], z.imag, atol=2e-2)
    assert np.array_equal(r[:, 64:], qf[:, 64:])
    # rotations preserve the pair norm (to bf16 rounding)
    assert np.allclose(r[:, :32] ** 2 + r[:, 32:64] ** 2, np.abs(z) ** 2, rtol=2e-2, atol=1e-3)


def test_argmax_known_answers(orc):
    # prototypes/test_argmax.ts:33-44
    V = 248320
    data = (np.sin(np.arange(V, dtype=np.float64)) * 10).astype(np.float32)
    data[123456] = 999.0
    assert orc.argmax(data) == (999.0, 123456)
    # ties: lowest index wins; NaN never wins; all -inf keeps index 0
    t = np.zeros(1000, np.float32); t[[17, 400, 999]] = 5.0
    assert orc.argmax(t) == (5.0, 17)
    t[3] = np.nan
    assert orc.argmax(t) == (5.0, 17)
    assert orc.argmax(np.full(8, -np.inf, np.float32))[1] == 0
    assert orc.argmax(np.array([-5.0, -3.0, -3.0, -9.0], np.float32)) == (-3.0, 1)


def test_embed(orc):
    E = np.arange(10 * 8, dtype=np.uint16).reshape(10, 8)
    assert np.array_equal(orc.embed(E, 7, 8), E[7])


# ------------------------------------------------------------------ GDN
def _gdn_inputs(g, Hg):
    dk = dv = 128
    conv = bf(g.standard_normal(3 * Hg * dk).astype(np.float32))
    z = bf(g.standard_normal(Hg * dv).astype(np.float32))
    A_log = (g.standard_normal(Hg) * 0.5).astype(np.float32)
    dt_bias = bf(g.standard_normal(Hg).astype(np.float32))
    a_p = g.standard_normal(Hg).astype(np.float32); b_p = g.standard_normal(Hg).astype(np.float32)
    norm_w = (1 + 0.1 * g.standard_normal(dv)).astype(np.float32)
    S = (g.standard_normal((Hg, dk, dv)) * 0.02).astype(np.float32)
    return conv, z, A_log, dt_bias, a_p, b_p, norm_w, S


def _gdn_f64(conv, z, A_log, dt_bias, a_p, b_p, norm_w, S, Hg):
    """float64 restatement of src/emitters.ts:75-120 written as matrix algebra."""
    dk = dv = 128
    c = f32(conv).astype(np.float64).reshape(3, Hg, dk)
    q, k, v = c[0], c[1], c[2]
    qh = q / np.sqrt((q * q).sum(1, keepdims=True) + 1e-6) / np.sqrt(dk)
    kh = k / np.sqrt((k * k).sum(1, keepdims=True) + 1e-6)
    sp = np.log1p(np.exp(a_p.astype(np.float64) + f32(dt_bias).astype(np.float64)))
    gdec = np.exp(-np.exp(A_log.astype(np.float64)) * sp)
    beta = 1 / (1 + np.exp(-b_p.astype(np.float64)))
    Sd = S.astype(np.float64) * gdec[:, None, None]
    kS = np.einsum("hk,hkv->hv", kh, Sd)
    delta = (v - kS) * beta[:, None]
    Sn = Sd + kh[:, :, None] * delta[:, None, :]
    o = np.einsum("hk,hkv->hv", qh, Sn)
    on = o / np.sqrt((o * o).mean(1, keepdims=True) + 1e-6) * norm_w.astype(np.float64)
    zf = f32(z).astype(np.float64).reshape(Hg, dv)
    return on * zf / (1 + np.exp(-zf)), Sn


def test_gdn_step_vs_float64(orc):
    g = synth.rng(30)
    Hg = 4
    args = _gdn_inputs(g, Hg)
    out, Sn = orc.gdn_step(*args, Hg)
    ref_o, ref_S = _gdn_f64(*args, Hg)
    assert np.abs(Sn - ref_S).max() <= 1e-5 * np.abs(ref_S).max()
    _close_bf16(out.reshape(Hg, 128), ref_o)


def test_gdn_invariants(orc):
    g = synth.rng(31)
    Hg = 3
    conv, z, A_log, dt_bias, a_p, b_p, norm_w, S = _gdn_inputs(g, Hg)
    # beta -> 0 (b = -inf): S' = decay * S exactly, elementwise in f32
    _, Sn = orc.gdn_step(conv, z, A_log, dt_bias, a_p, np.full(Hg, -np.inf, np.float32), norm_w, S, Hg)
    sp = np.log2(1 + np.exp((a_p + f32(dt_bias)).astype(np.float32))).astype(np.float32) * np.float32(np.log(2))
    dec = np.exp(-(np.exp(A_log) * sp)).astype(np.float32)
    assert np.allclose(Sn, S * dec[:, None, None], rtol=3e-6, atol=0)
    # S = 0, beta = 1 (b = +inf): S' = k^ (x) v and o = (q^ . k^) v  (prototypes/compare.ts seq=1 identity)
    core_q = bf(g.standard_normal(Hg * 128).astype(np.float32))
    core_k = bf(g.standard_normal(Hg * 128).astype(np.float32))
    core_v = bf(g.standard_normal(Hg * 128).astype(np.float32))
    o, Sn = orc.gdn_core(core_q, core_k, core_v, np.zeros(Hg, np.float32), np.ones(Hg, np.float32),
                         np.zeros((Hg, 128, 128), np.float32), Hg)
    qf = f32(core_q).reshape(Hg, 128).astype(np.float64); kf = f32(core_k).reshape(Hg, 128).astype(np.float64)
    vf = f32(core_v).reshape(Hg, 128).astype(np.float64)
    assert np.allclose(Sn, kf[:, :, None] * vf[:, None, :], rtol=1e-6, atol=1e-7)
    _close_bf16(o.reshape(Hg, 128), (qf * kf).sum(1, keepdims=True) * vf)


def test_gdn_core_vs_refgdn_loop(orc):
    """prototypes/gdn_gated.ts:67-88 refGDN as nested loops, float64, T = 3 steps chained
    through the single-step core (kb = k*beta, vb = v*beta as that file prepares them)."""
    g = synth.rng(32)
    Hg, dk, dv, T = 2, 128, 128, 3
    S = np.zeros((Hg, dk, dv)); S_orc = np.zeros((Hg, dk, dv), np.float32)
    for _ in range(T):
        q = bf((g.random(Hg * dk) * 0.6 - 0.3).astype(np.float32))
        k = bf((g.random(Hg * dk) * 0.6 - 0.3).astype(np.float32))
        v = bf((g.random(Hg * dv) * 0.6 - 0.3).astype(np.float32))
        beta = (g.random(Hg) * 0.8 + 0.1).astype(np.float32)
        dec = (0.95 + g.random(Hg) * 0.04).astype(np.float32)
        gl = np.log(dec).astype(np.float32)
        o_orc, S_orc = orc.gdn_core(q, k, v, gl, beta, S_orc, Hg)
        O = np.zeros((Hg, dv))
        for h in range(Hg):
            qq = f32(q).astype(np.float64)[h * dk:(h + 1) * dk]
            kk = f32(k).astype(np.float64)[h * dk:(h + 1) * dk]
            vv = f32(v).astype(np.float64)[h * dv:(h + 1) * dv]
            kb = kk * beta[h]; vb = vv * beta[h]
            S[h] *= np.exp(np.float64(gl[h]))
            kS = np.array([sum(kb[i] * S[h, i, d] for i in range(dk)) for d in range(dv)])
            delta = vb - kS
            for i in range(dk):
                S[h, i] += kk[i] * delta
            O[h] = [sum(qq[i] * S[h, i, d] for i in range(dk)) for d in range(dv)]
        assert np.abs(S_orc - S).max() <= 1e-5 * max(np.abs(S).max(), 1e-3)
        _close_bf16(o_orc.reshape(Hg, dv), O)


# ------------------------------------------------------------------ attention
def _attn_f64(q, kc, vc, bt, ctx, B, NH, NKV, HD, ps):
    G = NH // NKV
    out = np.zeros((B, NH, HD)); lse = np.zeros((B, NH))
    qf = f32(q).astype(np.float64).reshape(B, NH, HD)
    for b in range(B):
        n = int(ctx[b]); pages = bt[b, :(n + ps - 1) // ps]
        K = f32(kc[pages]).astype(np.float64).transpose(1, 0, 2, 3).reshape(NKV, -1, HD)[:, :n]
        V = f32(vc[pages]).astype(np.float64).transpose(1, 0, 2, 3).reshape(NKV, -1, HD)[:, :n]
        for h in range(NH):
            s = K[h // G] @ qf[b, h] / np.sqrt(HD)
            m = s.max(); p = np.exp(s - m)
            out[b, h] = p @ V[h // G] / p.sum()
            lse[b, h] = m + np.log(p.sum())
    return out, lse


def test_attn_vs_float64_softmax(orc):
    g = synth.rng(40)
    B, L, NH, NKV, HD, ps = 3, 200, 16, 2, 256, 16
    kc, vc, bt, ctx = synth.paged_kv_random(g, B, L, NKV, HD, ps)
    ctx[0] = 1; ctx[1] = 17                                 # one-token and ragged-page cases
    q = bf(g.standard_normal((B, NH, HD)).astype(np.float32))
    out, lse = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, NH, NKV, HD, ps)
    ref_o, ref_l = _attn_f64(q, kc, vc, bt, ctx, B, NH, NKV, HD, ps)
    _close_bf16(out, ref_o, 1e-2)
    assert np.allclose(lse, ref_l, rtol=1e-5, atol=1e-5)
    # len == 1: o = v of that token, lse = its score
    page0 = bt[0, 0]
    for h in range(NH):
        assert np.array_equal(out[0, h], vc[page0, h // 8, 0])
        s = (f32(q[0, h]).astype(np.float64) @ f32(kc[page0, h // 8, 0]).astype(np.float64)) / 16.0
        assert abs(lse[0, h] - s) < 1e-5 * max(1, abs(s))


def test_attn_page_permutation_invariance(orc):
    g = synth.rng(41)
    B, L, NH, NKV, HD, ps = 2, 300, 16, 2, 256, 16
    kc, vc, bt, ctx = synth.paged_kv_random(g, B, L, NKV, HD, ps)
    q = bf(g.standard_normal((B, NH, HD)).astype(np.float32))
    o1, l1 = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, NH, NKV, HD, ps)
    perm = g.permutation(kc.shape[0])
    inv = np.empty_like(perm); inv[perm] = np.arange(perm.size)
    o2, l2 = orc.attn_decode_paged(q, kc[perm], vc[perm], inv[bt].astype(np.int32), ctx, B, NH, NKV, HD, ps)
    assert np.array_equal(o1, o2) and np.array_equal(l1, l2)


def test_attn_gate_and_kv_append(orc):
    g = synth.rng(42)
    B, NH, NKV, HD, ps = 1, 16, 2, 256, 16
    kc, vc, bt, ctx = synth.paged_kv_random(g, B, 64, NKV, HD, ps)
    ctx[0] = 40
    k = bf(g.standard_normal((NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((NKV, HD)).astype(np.float32))
    orc.kv_append(k, v, kc, vc, bt[0], 40, NKV, HD, ps)
    pg = bt[0, 40 // ps]
    assert np.array_equal(kc[pg, :, 40 % ps], k) and np.array_equal(vc[pg, :, 40 % ps], v)
    ctx[0] = 41
    q = bf(g.standard_normal((B, NH, HD)).astype(np.float32))
    qgate = bf(g.standard_normal((NH, 2, HD)).astype(np.float32))        # [q | gate] per head as q_proj emits
    o_plain, _ = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, NH, NKV, HD, ps)
    o_gate, _ = orc.attn_decode_paged(q, kc, vc, bt, ctx, B, NH, NKV, HD, ps,
                                      gate=qgate.ravel()[HD:], gate_bstride=0, gate_hstride=2 * HD)
    ref_o, _ = _attn_f64(q, kc, vc, bt, ctx, B, NH, NKV, HD, ps)
    gt = f32(qgate[:, 1]).astype(np.float64)
    _close_bf16(o_gate[0], ref_o[0] / (1 + np.exp(-gt)), 1e-2)
    _close_bf16(o_plain[0], ref_o[0], 1e-2)
