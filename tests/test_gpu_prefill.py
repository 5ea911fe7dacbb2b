"""Prompt processing on the GPU against token-by-token runs of the CPU checker.

conv1d_prefill and gdn_prefill must give the bits of T single-token steps; fa2_prefill must leave the same cache
bytes and attention outputs with equal bits (exact=0: within 2e-2); the whole prefill must leave the state and the last token's logits of a
token-by-token run (the checker continues from the GPU's attention outputs, as in the decode tests), and decoding
must continue from that state as if every prompt token had been decoded."""
import numpy as np
import pytest

from bunker_amd import model, prefill, runner, synth, synth_model
from bunker_amd import runtime as rt
from bunker_amd.model import TINY

pytestmark = pytest.mark.gpu

bf = synth.f32_to_bf16
f32 = synth.bf16_to_f32


def _launch(spec, args):
    k = rt.compileAndLoad(spec)
    rc = rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], args)
    assert rc == 0, rt.last_error()
    rt.cuSync()


@pytest.mark.parametrize("T", [1, 2, 3, 7, 40])
def test_conv1d_prefill_is_T_decode_steps(orc, T):
    print(f"conv1d_prefill T={T}", flush=True)
    g = synth.rng(800 + T)
    C = 768
    x = bf(g.standard_normal((T, C)).astype(np.float32))
    st = bf(g.standard_normal((3, C)).astype(np.float32))
    w = bf((g.standard_normal((C, 4)) * 0.5).astype(np.float32))
    dx, dst, dw = rt.to_device(x), rt.to_device(st), rt.to_device(w)
    dout = rt.cuAlloc(T * C * 2)
    _launch(f"conv1d_prefill QKVD={C} T={T}", [dx, dst, dw, dout, dst])        # state updated in place
    got = rt.from_device(dout, (T, C), np.uint16); gst = rt.from_device(dst, (3, C), np.uint16)
    s = st
    for t in range(T):
        ref, s = orc.conv1d_decode(x[t], s, w)
        assert np.array_equal(got[t], ref), t
    assert np.array_equal(gst, s)
    for p in (dx, dst, dw, dout):
        rt.cuFree(p)


@pytest.mark.parametrize("Hg,T", [(2, 1), (3, 5), (4, 32), (16, 33)])
def test_gdn_prefill_is_T_decode_steps(orc, Hg, T):
    print(f"gdn_prefill Hg={Hg} T={T}", flush=True)
    g = synth.rng(820 + Hg + T)
    C = 3 * Hg * 128
    conv = bf(g.standard_normal((T, C)).astype(np.float32))
    z = bf(g.standard_normal((T, Hg * 128)).astype(np.float32))
    A_log = g.uniform(-2, 1, Hg).astype(np.float32)
    dt_bias = bf(g.standard_normal(Hg).astype(np.float32))
    a_p = g.standard_normal((T, Hg)).astype(np.float32); b_p = g.standard_normal((T, Hg)).astype(np.float32)
    norm_w = (1 + 0.1 * g.standard_normal(128)).astype(np.float32)
    S = (g.standard_normal((Hg, 128, 128)) * 0.02).astype(np.float32)
    ptrs = [rt.to_device(a) for a in (conv, z, A_log, dt_bias, a_p, b_p, norm_w, S)]
    dout = rt.cuAlloc(T * Hg * 128 * 2)
    _launch(f"gdn_prefill LVH={Hg} T={T}", ptrs + [dout, ptrs[7]])                # S updated in place
    got = rt.from_device(dout, (T, Hg * 128), np.uint16); gS = rt.from_device(ptrs[7], S.shape, np.float32)
    s = S
    for t in range(T):
        ro, s = orc.gdn_step(conv[t], z[t], A_log, dt_bias, a_p[t], b_p[t], norm_w, s, Hg, rows_per_chain=16)
        assert np.array_equal(got[t], ro), t
    assert np.array_equal(gS.view(np.uint32), s.view(np.uint32))
    for p in ptrs + [dout]:
        rt.cuFree(p)


@pytest.mark.parametrize("Hg,T", [(2, 1), (3, 5), (2, 64), (4, 65), (3, 200), (16, 1024)])
def test_gdn_prefill_chunked_form_against_the_scan(Hg, T):
    """chunked=1 (chunks of 64 tokens, f32 matrix instruction) against the scan, which has the checker's bits: the
    state within 2e-5 of the largest state element, the bf16 outputs within one step of bf16 (2^-7 relative) — the two
    forms add the same f32 terms in different orders.  Covers a lone token, a partial chunk, exactly one chunk, a
    partial chunk behind full ones, and a 16-chunk run with strong and weak decays in the same head."""
    print(f"gdn_prefill chunked Hg={Hg} T={T}", flush=True)
    g = synth.rng(8200 + Hg + T)
    C = 3 * Hg * 128
    conv = bf(g.standard_normal((T, C)).astype(np.float32))
    z = bf(g.standard_normal((T, Hg * 128)).astype(np.float32))
    A_log = g.uniform(-2, 1, Hg).astype(np.float32)
    dt_bias = bf(g.standard_normal(Hg).astype(np.float32))
    a_p = (g.standard_normal((T, Hg)) * 2).astype(np.float32); b_p = g.standard_normal((T, Hg)).astype(np.float32)
    norm_w = (1 + 0.1 * g.standard_normal(128)).astype(np.float32)
    S = (g.standard_normal((Hg, 128, 128)) * 0.02).astype(np.float32)
    res = []
    for chunked in (0, 1):
        ptrs = [rt.to_device(a) for a in (conv, z, A_log, dt_bias, a_p, b_p, norm_w, S)]
        dout = rt.cuAlloc(T * Hg * 128 * 2)
        rt.cuMemset(dout, 0xff, T * Hg * 128 * 2)
        _launch(f"gdn_prefill LVH={Hg} T={T} chunked={chunked}", ptrs + [dout, ptrs[7]])
        res.append((f32(rt.from_device(dout, (T, Hg * 128), np.uint16)).astype(np.float64), rt.from_device(ptrs[7], S.shape, np.float32).astype(np.float64)))
        for p in ptrs + [dout]:
            rt.cuFree(p)
    (o0, S0), (o1, S1) = res
    assert np.isfinite(o1).all() and np.isfinite(S1).all()
    assert np.abs(S1 - S0).max() <= 2e-5 * np.abs(S0).max(), (np.abs(S1 - S0).max(), np.abs(S0).max())
    assert np.all(np.abs(o1 - o0) <= 2.0 ** -7 * np.abs(o0) + 1e-4), np.abs(o1 - o0).max()


def _gdn_inputs(g, Hg, T, decay_mix):
    C = 3 * Hg * 128
    conv = bf(g.standard_normal((T, C)).astype(np.float32))
    z = bf(g.standard_normal((T, Hg * 128)).astype(np.float32))
    A_log = g.uniform(-2, 1, Hg).astype(np.float32)
    dt_bias = bf(g.standard_normal(Hg).astype(np.float32))
    a_p = (g.standard_normal((T, Hg)) * 2).astype(np.float32); b_p = g.standard_normal((T, Hg)).astype(np.float32)
    if decay_mix:
        # strong and weak decays in the same run: head 0 barely decays (decay ~ 1 - 1e-4), head 1 loses most of its
        # state at every token (decay ~ e^-8), the others alternate between the two by token
        A_log[0] = -4.0; a_p[:, 0] = -4.0
        if Hg > 1:
            A_log[1] = 1.0; a_p[:, 1] = 3.0
        for h in range(2, Hg):
            a_p[::2, h] = -5.0; a_p[1::2, h] = 3.0
    norm_w = (1 + 0.1 * g.standard_normal(128)).astype(np.float32)
    S = (g.standard_normal((Hg, 128, 128)) * 0.02).astype(np.float32)
    return conv, z, A_log, dt_bias, a_p, b_p, norm_w, S


def _gdn_prefill_gpu(inputs, Hg, T, chunked):
    ptrs = [rt.to_device(a) for a in inputs]
    dout = rt.cuAlloc(T * Hg * 128 * 2)
    rt.cuMemset(dout, 0xff, T * Hg * 128 * 2)
    _launch(f"gdn_prefill LVH={Hg} T={T} chunked={chunked}", ptrs + [dout, ptrs[7]])
    out = rt.from_device(dout, (T, Hg * 128), np.uint16)
    S = rt.from_device(ptrs[7], inputs[7].shape, np.float32)
    for p in ptrs + [dout]:
        rt.cuFree(p)
    return out, S


@pytest.mark.parametrize("Hg,T,decay_mix", [(3, 200, False), (16, 1024, False), (4, 300, True)])
def test_gdn_prefill_both_forms_against_the_checker_chained_over_T(orc, Hg, T, decay_mix):
    """Scan and chunked form against the checker's single-token step chained over T tokens (the multi-token host loop of
    prototypes/gdn_gated.ts:67-88 refGDN, one token at a time).  Yardstick: the checker with both k-reductions
    accumulated in double (rows_per_chain=0).  Both GPU forms: state within 1e-4 of the largest state element per
    head, bf16 outputs within 2e-2 max-abs (plus one bf16 step for the large ones).  At T = 200 the scan must also
    return the bytes of the checker in the canonical f32 order (rows_per_chain=16) — past the 16-token lookahead of
    its LDS staging and past a 64-token chunk boundary."""
    print(f"gdn_prefill vs checker Hg={Hg} T={T} decay_mix={decay_mix}", flush=True)
    g = synth.rng(8300 + Hg + T)
    inp = _gdn_inputs(g, Hg, T, decay_mix)
    conv, z, A_log, dt_bias, a_p, b_p, norm_w, S = inp
    ref_o = np.empty((T, Hg * 128), np.uint16)
    s = S
    for t in range(T):
        ref_o[t], s = orc.gdn_step(conv[t], z[t], A_log, dt_bias, a_p[t], b_p[t], norm_w, s, Hg, rows_per_chain=0)
    ref_S = s.astype(np.float64); ro = f32(ref_o).astype(np.float64)
    canon = None
    if T <= 300:
        canon_o = np.empty_like(ref_o); s = S
        for t in range(T):
            canon_o[t], s = orc.gdn_step(conv[t], z[t], A_log, dt_bias, a_p[t], b_p[t], norm_w, s, Hg, rows_per_chain=16)
        canon = (canon_o, s)
    for chunked in (0, 1):
        out, gS = _gdn_prefill_gpu(inp, Hg, T, chunked)
        assert not (out == 0xffff).any(), "an output row was left unwritten"
        o = f32(out).astype(np.float64)
        assert np.isfinite(o).all() and np.isfinite(gS).all()
        for h in range(Hg):
            scale = np.abs(ref_S[h]).max()
            err = np.abs(gS[h].astype(np.float64) - ref_S[h]).max()
            assert err <= 1e-4 * scale, (chunked, h, err, scale)
        d = np.abs(o - ro)
        assert np.all(d <= 2e-2 + 2.0 ** -7 * np.abs(ro)), (chunked, d.max(), np.unravel_index(d.argmax(), d.shape))
        if chunked == 0 and canon is not None:
            assert np.array_equal(out, canon[0]), "scan output bytes differ from the checker's canonical order"
            assert np.array_equal(gS.view(np.uint32), canon[1].view(np.uint32)), "scan state bits differ"


@pytest.mark.parametrize("T,pos0,splits", [(6, 0, 0), (37, 12, 0), (37, 60, 3), (2, 15, 2)])
def test_fa2_prefill_token_pairs_return_the_single_row_bits(orc, T, pos0, splits):
    """The matrix-instruction form (exact=0): two consecutive tokens per workgroup (their heads side by side in the 16 columns of the products, each column
    masked to its own length) against one token per workgroup: the same output and cache bytes."""
    print(f"fa2_prefill pairs T={T} pos0={pos0} splits={splits}", flush=True)
    g = synth.rng(870 + T + pos0)
    NH, NKV, HD, HALF, MAXL = 16, 2, 256, 32, 128
    pages = MAXL // 16
    cos_t, sin_t = orc.rope_tables(MAXL, 64, 1e7)
    kc = bf(g.standard_normal((pages, NKV, 16, HD)).astype(np.float32))
    vc = bf(g.standard_normal((pages, NKV, 16, HD)).astype(np.float32))
    qgate = bf(g.standard_normal((T, NH, 2, HD)).astype(np.float32))
    k = bf(g.standard_normal((T, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((T, NKV, HD)).astype(np.float32))
    qw = bf((g.standard_normal(HD) * 0.1).astype(np.float32)); kw = bf((g.standard_normal(HD) * 0.1).astype(np.float32))
    table = g.permutation(pages).astype(np.int32)
    pos = (pos0 + np.arange(T)).astype(np.int32)
    ptrs = [rt.to_device(a) for a in (qgate, k, v, qw, kw, cos_t, sin_t, pos, table)]
    res = []
    for pair in (0, 1):
        dkc, dvc = rt.to_device(kc), rt.to_device(rt.v_pages_to_device_layout(vc))
        dout = rt.cuAlloc(T * NH * HD * 2)
        rt.cuMemset(dout, 0xff, T * NH * HD * 2)
        _launch(f"fa2_prefill HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} ROT_HALF={HALF} T={T} pair={pair} exact=0 tiled=0" + (f" splits={splits}" if splits else ""),
                ptrs + [dkc, dvc, dout])
        res.append((rt.from_device(dout, (T, NH, HD), np.uint16), rt.from_device(dkc, kc.shape, np.uint16),
                    rt.from_device(dvc, (pages, NKV, HD, 16), np.uint16)))
        for p in (dkc, dvc, dout):
            rt.cuFree(p)
    for a, b in zip(res[0], res[1]):
        assert np.array_equal(a, b)
    assert not np.any(res[1][0] == 0xffff)
    for p in ptrs:
        rt.cuFree(p)


@pytest.mark.parametrize("exact", [1, 0])
@pytest.mark.parametrize("T,pos0", [(1, 0), (5, 0), (37, 12)])
def test_fa2_prefill_appends_and_attends_causally(orc, T, pos0, exact):
    """exact=1 (the default): every output row has the checker's bits; exact=0: within 2e-2."""
    print(f"fa2_prefill T={T} pos0={pos0} exact={exact}", flush=True)
    g = synth.rng(840 + T)
    NH, NKV, HD, HALF, MAXL = 16, 2, 256, 32, 128
    pages = MAXL // 16
    seq = 1                                       # the second sequence of a two-sequence cache
    cos_t, sin_t = orc.rope_tables(MAXL, 64, 1e7)
    kc = bf(g.standard_normal((2 * pages, NKV, 16, HD)).astype(np.float32))
    vc = bf(g.standard_normal((2 * pages, NKV, 16, HD)).astype(np.float32))
    qgate = bf(g.standard_normal((T, NH, 2, HD)).astype(np.float32))
    k = bf(g.standard_normal((T, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((T, NKV, HD)).astype(np.float32))
    qw = bf((g.standard_normal(HD) * 0.1).astype(np.float32)); kw = bf((g.standard_normal(HD) * 0.1).astype(np.float32))
    table = (seq * pages + np.arange(pages)).astype(np.int32)
    pos = (pos0 + np.arange(T)).astype(np.int32)
    dkc, dvc = rt.to_device(kc), rt.to_device(rt.v_pages_to_device_layout(vc))
    dout = rt.cuAlloc(T * NH * HD * 2)
    ptrs = [rt.to_device(a) for a in (qgate, k, v, qw, kw, cos_t, sin_t, pos, table)]
    _launch(f"fa2_prefill HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} ROT_HALF={HALF} T={T}" + ("" if exact else " exact=0"), ptrs + [dkc, dvc, dout])
    out = rt.from_device(dout, (T, NH, HD), np.uint16)
    worst = 0.0
    for t in range(T):
        qn = orc.rope(orc.headnorm(qgate[t].ravel(), qw, NH, HD, 2 * HD), cos_t, sin_t, pos[t], NH, HD, HALF).reshape(1, NH, HD)
        kn = orc.rope(orc.headnorm(k[t].ravel(), kw, NKV, HD, HD), cos_t, sin_t, pos[t], NKV, HD, HALF)
        orc.kv_append(kn.reshape(NKV, HD), v[t], kc, vc, table, pos[t], NKV, HD, 16)
        ro, _ = orc.attn_decode_paged(qn, kc, vc, table[None], np.array([pos[t] + 1], np.int32), 1, NH, NKV, HD, 16,
                                      gate=qgate[t].ravel()[HD:], gate_bstride=0, gate_hstride=2 * HD)
        worst = max(worst, float(np.abs(f32(out[t]).astype(np.float64) - f32(ro[0])).max()))
    assert worst <= (0.0 if exact else 2e-2), worst
    kc_d = rt.from_device(dkc, kc.shape, np.uint16)
    vc_d = rt.from_device(dvc, (2 * pages, NKV, HD, 16), np.uint16).transpose(0, 1, 3, 2)
    assert np.array_equal(kc_d, kc) and np.array_equal(vc_d, vc)
    for p in ptrs + [dkc, dvc, dout]:
        rt.cuFree(p)


@pytest.mark.parametrize("NH,NKV,T,pos0", [(16, 2, 200, 70), (16, 2, 64, 0), (8, 2, 97, 33), (4, 4, 130, 5), (16, 1, 50, 17), (4, 2, 129, 0),
                                            (16, 16, 150, 20)])      # (16 KV heads: two groups of workgroups per XCD)
def test_fa2_prefill_tiled_attention_against_the_checker(orc, NH, NKV, T, pos0):
    """exact=0 runs the query-tile x K/V-tile kernel (bf16 matrix cores): every row within 2e-2 of the f64 checker, for
    every group size it serves, ragged last query tile, a context that starts in the middle of a K/V tile, a permuted page
    table, and NaN bit patterns in the cache behind the prompt (they must not reach any output).  The caches get the
    same bytes as with exact=1 (the preparation is the same kernel)."""
    print(f"fa2_prefill tiled NH={NH} NKV={NKV} T={T} pos0={pos0}", flush=True)
    g = synth.rng(880 + NH + T)
    HD, HALF, MAXL = 256, 32, 512
    pages = MAXL // 16
    cos_t, sin_t = orc.rope_tables(MAXL, 64, 1e7)
    kc = bf(g.standard_normal((pages, NKV, 16, HD)).astype(np.float32))
    vc = bf(g.standard_normal((pages, NKV, 16, HD)).astype(np.float32))
    table = g.permutation(pages).astype(np.int32)
    end = pos0 + T
    for tok in range(end, MAXL):                   # behind the prompt: not numbers
        kc[table[tok // 16], :, tok % 16, :] = 0x7fc0
        vc[table[tok // 16], :, tok % 16, :] = 0xffc1
    qgate = bf(g.standard_normal((T, NH, 2, HD)).astype(np.float32))
    k = bf(g.standard_normal((T, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((T, NKV, HD)).astype(np.float32))
    qw = bf((g.standard_normal(HD) * 0.1).astype(np.float32)); kw = bf((g.standard_normal(HD) * 0.1).astype(np.float32))
    pos = (pos0 + np.arange(T)).astype(np.int32)
    ptrs = [rt.to_device(a) for a in (qgate, k, v, qw, kw, cos_t, sin_t, pos, table)]
    outs = {}
    for tiled in (1, 0):
        dkc, dvc = rt.to_device(kc), rt.to_device(rt.v_pages_to_device_layout(vc))
        dout = rt.cuAlloc(T * NH * HD * 2)
        rt.cuMemset(dout, 0xff, T * NH * HD * 2)
        _launch(f"fa2_prefill HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} ROT_HALF={HALF} T={T} exact=0 tiled={tiled}", ptrs + [dkc, dvc, dout])
        outs[tiled] = rt.from_device(dout, (T, NH, HD), np.uint16)
        kc_d = rt.from_device(dkc, kc.shape, np.uint16)
        vc_d = rt.from_device(dvc, (pages, NKV, HD, 16), np.uint16).transpose(0, 1, 3, 2)
        for p in (dkc, dvc, dout):
            rt.cuFree(p)
    assert not np.any(outs[1] == 0xffff)            # every row written, none of them NaN
    worst = 0.0
    for t in range(T):
        qn = orc.rope(orc.headnorm(qgate[t].ravel(), qw, NH, HD, 2 * HD), cos_t, sin_t, pos[t], NH, HD, HALF).reshape(1, NH, HD)
        kn = orc.rope(orc.headnorm(k[t].ravel(), kw, NKV, HD, HD), cos_t, sin_t, pos[t], NKV, HD, HALF)
        orc.kv_append(kn.reshape(NKV, HD), v[t], kc, vc, table, pos[t], NKV, HD, 16)
        ro, _ = orc.attn_decode_paged(qn, kc, vc, table[None], np.array([pos[t] + 1], np.int32), 1, NH, NKV, HD, 16,
                                      gate=qgate[t].ravel()[HD:], gate_bstride=0, gate_hstride=2 * HD)
        worst = max(worst, float(np.abs(f32(outs[1][t]).astype(np.float64) - f32(ro[0])).max()))
    assert worst <= 2e-2, worst
    assert np.array_equal(kc_d, kc) and np.array_equal(vc_d, vc)
    assert np.abs(f32(outs[1]).astype(np.float64) - f32(outs[0])).max() <= 2e-2
    for p in ptrs:
        rt.cuFree(p)


def test_fa2_prefill_tiled_attention_rows_in_any_order_and_a_long_context(orc):
    """The tiled kernel takes each row's length from pos[t] alone: rows whose positions are shuffled (every token is
    appended before any row attends, so row t sees all tokens at positions <= pos[t]) and a chunk far into a long
    cache (8000 tokens in front of it: 126 K/V tiles per workgroup) agree with the checker row by row."""
    print("fa2_prefill tiled shuffled / long", flush=True)
    g = synth.rng(8877)
    NH, NKV, HD, HALF = 16, 2, 256, 32
    for MAXL, T, pos0, shuffled in ((256, 90, 20, True), (8192, 48, 8000, False)):
        pages = MAXL // 16
        cos_t, sin_t = orc.rope_tables(MAXL, 64, 1e7)
        kc = bf(g.standard_normal((pages, NKV, 16, HD)).astype(np.float32))
        vc = bf(g.standard_normal((pages, NKV, 16, HD)).astype(np.float32))
        table = g.permutation(pages).astype(np.int32)
        qgate = bf(g.standard_normal((T, NH, 2, HD)).astype(np.float32))
        k = bf(g.standard_normal((T, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((T, NKV, HD)).astype(np.float32))
        qw = bf((g.standard_normal(HD) * 0.1).astype(np.float32)); kw = bf((g.standard_normal(HD) * 0.1).astype(np.float32))
        pos = (pos0 + (g.permutation(T) if shuffled else np.arange(T))).astype(np.int32)
        ptrs = [rt.to_device(a) for a in (qgate, k, v, qw, kw, cos_t, sin_t, pos, table)]
        dkc, dvc = rt.to_device(kc), rt.to_device(rt.v_pages_to_device_layout(vc))
        dout = rt.cuAlloc(T * NH * HD * 2)
        _launch(f"fa2_prefill HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} ROT_HALF={HALF} T={T} exact=0", ptrs + [dkc, dvc, dout])
        out = rt.from_device(dout, (T, NH, HD), np.uint16)
        for t in range(T):                              # all appends first, as the op does
            kn = orc.rope(orc.headnorm(k[t].ravel(), kw, NKV, HD, HD), cos_t, sin_t, pos[t], NKV, HD, HALF)
            orc.kv_append(kn.reshape(NKV, HD), v[t], kc, vc, table, pos[t], NKV, HD, 16)
        worst = 0.0
        for t in range(T):
            qn = orc.rope(orc.headnorm(qgate[t].ravel(), qw, NH, HD, 2 * HD), cos_t, sin_t, pos[t], NH, HD, HALF).reshape(1, NH, HD)
            ro, _ = orc.attn_decode_paged(qn, kc, vc, table[None], np.array([pos[t] + 1], np.int32), 1, NH, NKV, HD, 16,
                                          gate=qgate[t].ravel()[HD:], gate_bstride=0, gate_hstride=2 * HD)
            worst = max(worst, float(np.abs(f32(out[t]).astype(np.float64) - f32(ro[0])).max()))
        assert worst <= 2e-2, (MAXL, worst)
        for p in ptrs + [dkc, dvc, dout]:
            rt.cuFree(p)


def test_fa2_prefill_tiled_attention_cut_along_the_context(orc):
    """A launch with fewer workgroups than CUs is cut along K/V into 2..4 runs whose unnormalised rows a second kernel
    joins (tuning key prefill_ksplit; 0 = chosen from the shape, here 4).  Every cut agrees with the checker row by row,
    also where a run of a short row holds no token at all (rows of 1501..1540 tokens in runs of 6 tiles), and with the
    uncut launch to a few bf16 steps."""
    print("fa2_prefill tiled, cut along K/V", flush=True)
    g = synth.rng(4242)
    NH, NKV, HD, HALF, MAXL, T, pos0 = 16, 2, 256, 32, 2048, 40, 1500
    pages = MAXL // 16
    cos_t, sin_t = orc.rope_tables(MAXL, 64, 1e7)
    kc = bf(g.standard_normal((pages, NKV, 16, HD)).astype(np.float32))
    vc = bf(g.standard_normal((pages, NKV, 16, HD)).astype(np.float32))
    table = g.permutation(pages).astype(np.int32)
    for tok in range(pos0 + T, MAXL):                  # behind the prompt: not numbers
        kc[table[tok // 16], :, tok % 16, :] = 0x7fc0
        vc[table[tok // 16], :, tok % 16, :] = 0xffc1
    qgate = bf(g.standard_normal((T, NH, 2, HD)).astype(np.float32))
    k = bf(g.standard_normal((T, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((T, NKV, HD)).astype(np.float32))
    qw = bf((g.standard_normal(HD) * 0.1).astype(np.float32)); kw = bf((g.standard_normal(HD) * 0.1).astype(np.float32))
    pos = (pos0 + np.arange(T)).astype(np.int32)
    pos[3] = 70                                        # one row far shorter than the rest: most runs hold none of its tokens
    ptrs = [rt.to_device(a) for a in (qgate, k, v, qw, kw, cos_t, sin_t, pos, table)]
    outs = {}
    try:
        for ks in (1, 2, 3, 4, 0):
            rt.tune_set("prefill_ksplit", ks)
            dkc, dvc = rt.to_device(kc), rt.to_device(rt.v_pages_to_device_layout(vc))
            dout = rt.cuAlloc(T * NH * HD * 2)
            rt.cuMemset(dout, 0xff, T * NH * HD * 2)
            _launch(f"fa2_prefill HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} ROT_HALF={HALF} T={T} exact=0", ptrs + [dkc, dvc, dout])
            outs[ks] = rt.from_device(dout, (T, NH, HD), np.uint16)
            for p in (dkc, dvc, dout):
                rt.cuFree(p)
    finally:
        rt.tune_set("prefill_ksplit", 0)
    order = np.argsort(pos, kind="stable")              # the op appends every token before any row attends
    for t in range(T):
        kn = orc.rope(orc.headnorm(k[t].ravel(), kw, NKV, HD, HD), cos_t, sin_t, pos[t], NKV, HD, HALF)
        orc.kv_append(kn.reshape(NKV, HD), v[t], kc, vc, table, pos[t], NKV, HD, 16)
    for ks, out in outs.items():
        assert not np.any(out == 0xffff), ks
        worst = 0.0
        for t in order:
            qn = orc.rope(orc.headnorm(qgate[t].ravel(), qw, NH, HD, 2 * HD), cos_t, sin_t, pos[t], NH, HD, HALF).reshape(1, NH, HD)
            ro, _ = orc.attn_decode_paged(qn, kc, vc, table[None], np.array([pos[t] + 1], np.int32), 1, NH, NKV, HD, 16,
                                          gate=qgate[t].ravel()[HD:], gate_bstride=0, gate_hstride=2 * HD)
            worst = max(worst, float(np.abs(f32(out[t]).astype(np.float64) - f32(ro[0])).max()))
        assert worst <= 2e-2, (ks, worst)
        assert np.abs(f32(out).astype(np.float64) - f32(outs[1])).max() <= 2e-2, ks
    for p in ptrs:
        rt.cuFree(p)


@pytest.mark.parametrize("n_prompt,chunk", [(23, 8), (9, 16)])
def test_prefill_then_decode_equals_token_by_token(orc, n_prompt, chunk):
    """TINY model, two sequences in the cache; the prompt goes to sequence 1 in chunks (with a shorter last chunk),
    then both the checker and the GPU decode 3 more tokens from the state the prompt left."""
    print(f"prefill n={n_prompt} chunk={chunk}", flush=True)
    from oracle.model_ref import RefModel
    D = TINY
    B, seq = 2, 1
    W = synth_model.synth_weights(D, seed=31)
    S = synth_model.synth_state(D, B, seed=32)
    for key in S:                                 # a fresh sequence: no conv history, S = 0
        if key.endswith("conv_state") or key.endswith("s_state"):
            S[key][seq] = 0
    g = model.buildModelGraph(D, B)
    env = runner.DecodeEnv(g, W, synth_model.device_state(S), inplace_state=True)
    prompt = synth.rng(33).integers(0, D.VOCAB, n_prompt).astype(np.int32)
    captured = {}
    pf = prefill.Prefill(D, env, chunk=chunk,
                         on_attention=lambda layer, first, rows: captured.setdefault(layer, {}).update({first + i: r for i, r in enumerate(rows)}))
    tok, val = pf.run(prompt, seq=seq, pos0=0)
    glogits = rt.from_device(pf.d_logits, (D.VOCAB,), np.float32)

    ref = RefModel(D, W, {k: np.asarray(v)[[seq]] for k, v in S.items()}, batch=1)
    for t in range(n_prompt):
        inj = {l: captured[l][t][None] for l in captured}
        idx, rv, rlogits = ref.step([prompt[t]], [t], attn_override=inj)
    assert max(ref.attn_err) == 0.0, max(ref.attn_err)         # double-precision attention: the checker's bits
    assert np.array_equal(glogits.view(np.uint32), rlogits[0].view(np.uint32)), \
        f"{int((glogits != rlogits[0]).sum())} logits differ, worst {np.abs(glogits - rlogits[0]).max():.3e}"
    assert tok == int(idx[0]) and np.float32(val).view(np.uint32) == rv[0].view(np.uint32)
    for l in range(D.NL):
        p = f"model.layers.{l}"
        if not D.is_full_attention(l):
            Sg = env.read_state(f"{p}.s_state", (B, D.LVH, 128, 128), np.float32)
            assert np.array_equal(Sg[seq].view(np.uint32), ref.S[f"{p}.s_state"][0].view(np.uint32)), p
            assert np.array_equal(Sg[0], S[f"{p}.s_state"][0]), "the other sequence's state was touched"
            cg = env.read_state(f"{p}.conv_state", (B, 3, D.QKVD), np.uint16)
            assert np.array_equal(cg[seq], ref.S[f"{p}.conv_state"][0]), p
        else:
            kg = env.read_state(f"{p}.kv_k", (B,) + ref.S[f"{p}.kv_k"].shape[1:], np.uint16)
            assert np.array_equal(kg[seq], ref.S[f"{p}.kv_k"][0]) and np.array_equal(kg[0], np.asarray(S[f"{p}.kv_k"])[0]), p
            vg = env.read_state(f"{p}.kv_v", (B, D.MAX_LEN // 16, D.NKV, D.HD, 16), np.uint16).swapaxes(-1, -2)
            assert np.array_equal(vg[seq], ref.S[f"{p}.kv_v"][0]), p
    pf.close()

    # decode continues from the prompt's state: sequence 1 from its first generated token at pos n_prompt
    steps = 3
    loop = runner.DeviceLoop(g, env, B, [7, tok], [40, n_prompt], max_steps=steps, partition=runner.fusedPartition(g))
    fa_nodes = [n for n in g.nodes if n.op == "fa2_attn"]
    fa_layers = [l for l in range(D.NL) if D.is_full_attention(l)]
    toks, pos = np.array([tok], np.int32), np.array([n_prompt], np.int32)
    for step in range(steps):
        loop.step(1)
        rt.cuSync()
        inj = {l: rt.from_device(env.resolve(n.outputs[0].tensorName), (B, D.NH * D.HD), np.uint16)[[seq]]
               for l, n in zip(fa_layers, fa_nodes)}
        idx, rv, _ = ref.step(toks, pos, attn_override=inj)
        gt, gv = loop.tokens()
        assert gt[step][seq] == idx[0] and gv[step][seq].view(np.uint32) == rv[0].view(np.uint32), (step, gt[step], idx)
        toks, pos = idx, pos + 1
    assert max(ref.attn_err) == 0.0
    env.close()


@pytest.mark.parametrize("n_prompt,chunk", [(61, 8), (40, 16)])
def test_prefill_two_chunks_in_flight_equals_one(orc, n_prompt, chunk):
    """Two chunks in flight on two streams (each layer's state hand-over ordered by events) leave the same bytes as
    one chunk at a time: logits of the last prompt token, first token, and every state tensor."""
    print(f"prefill overlap n={n_prompt} chunk={chunk}", flush=True)
    D = TINY
    B, seq = 2, 1
    W = synth_model.synth_weights(D, seed=51)
    S = synth_model.synth_state(D, B, seed=52)
    prompt = synth.rng(53).integers(0, D.VOCAB, n_prompt).astype(np.int32)
    g = model.buildModelGraph(D, B)
    results = []
    for overlap in (False, True, True):
        env = runner.DecodeEnv(g, W, synth_model.device_state(S), inplace_state=True)
        pf = prefill.Prefill(D, env, chunk=chunk, overlap=overlap)
        tok, val = pf.run(prompt[:n_prompt // 2], seq=seq, pos0=0)            # two runs: the second continues the first
        tok, val = pf.run(prompt[n_prompt // 2:], seq=seq, pos0=n_prompt // 2)
        state = {"logits": rt.from_device(pf.d_logits, (D.VOCAB,), np.float32).view(np.uint32), "tok": tok,
                 "val": np.float32(val).view(np.uint32)}
        for l in range(D.NL):
            p = f"model.layers.{l}"
            if not D.is_full_attention(l):
                state[p + ".S"] = env.read_state(f"{p}.s_state", (B, D.LVH, 128, 128), np.float32).view(np.uint32)
                state[p + ".conv"] = env.read_state(f"{p}.conv_state", (B, 3, D.QKVD), np.uint16)
            else:
                state[p + ".k"] = env.read_state(f"{p}.kv_k", (B, D.MAX_LEN // 16, D.NKV, 16, D.HD), np.uint16)
                state[p + ".v"] = env.read_state(f"{p}.kv_v", (B, D.MAX_LEN // 16, D.NKV, D.HD, 16), np.uint16)
        results.append(state)
        pf.close()
        env.close()
    for other in results[1:]:
        for key, v in results[0].items():
            assert np.array_equal(v, other[key]), key


def test_prefill_in_the_chunked_and_tiled_forms_stays_close_to_the_exact_one():
    """A TINY-model prompt through the forms of the reference's prefill prototypes (fa2_prefill exact=0: tiled bf16
    attention; gdn_prefill chunked=1: chunks of 64 tokens in f32) against the default forms, which leave the bits of
    token-by-token decoding: the conv rows are the same bytes (that op has one form), the GDN states agree to 1e-3 of
    their largest element and the logits of the last prompt token to 0.05 — the differences are the rounding of
    attention weights to bf16 and the order of the f32 additions, carried through the layers by the bf16 activations."""
    print("prefill chunked/tiled vs exact", flush=True)
    from dataclasses import replace
    D = replace(TINY, MAX_LEN=256)
    B, seq, n_prompt, chunk = 2, 1, 150, 96
    W = synth_model.synth_weights(D, seed=61)
    S = synth_model.synth_state(D, B, seed=62)
    for key in S:
        if key.endswith("conv_state") or key.endswith("s_state"):
            S[key][seq] = 0
    prompt = synth.rng(63).integers(0, D.VOCAB, n_prompt).astype(np.int32)
    g = model.buildModelGraph(D, B)
    results = []
    for fast in (False, True):
        env = runner.DecodeEnv(g, W, synth_model.device_state(S), inplace_state=True)
        pf = prefill.Prefill(D, env, chunk=chunk, gdn_chunked=fast, attn_exact=not fast)
        tok, val = pf.run(prompt, seq=seq, pos0=0)
        state = {"logits": rt.from_device(pf.d_logits, (D.VOCAB,), np.float32).astype(np.float64), "tok": tok}
        for l in range(D.NL):
            p = f"model.layers.{l}"
            if not D.is_full_attention(l):
                state[p + ".S"] = env.read_state(f"{p}.s_state", (B, D.LVH, 128, 128), np.float32).astype(np.float64)
                state[p + ".conv"] = env.read_state(f"{p}.conv_state", (B, 3, D.QKVD), np.uint16)
        results.append(state)
        pf.close()
        env.close()
    exact, fast = results
    first_gdn = next(l for l in range(D.NL) if not D.is_full_attention(l))
    assert np.array_equal(exact[f"model.layers.{first_gdn}.conv"], fast[f"model.layers.{first_gdn}.conv"])     # same inputs, one form
    for key, v in exact.items():
        if key.endswith(".S"):
            assert np.abs(fast[key] - v).max() <= 1e-3 * np.abs(v).max(), (key, np.abs(fast[key] - v).max(), np.abs(v).max())
    assert np.isfinite(fast["logits"]).all()
    assert np.abs(fast["logits"] - exact["logits"]).max() <= 0.05, np.abs(fast["logits"] - exact["logits"]).max()
