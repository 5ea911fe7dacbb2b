"""GPU parity of the fused decode kernels against the node-by-node CPU checker.

A fused launch must give the bits of the sequence of graph nodes it replaces (rmsnorm -> gemm
[-> cast -> add | -> swiglu], conv1d -> gdn_delta_rule, qnorm/rope/knorm/ropek -> cache append):
kernels and checker share the arithmetic rules, so every comparison here is for equality."""
import numpy as np
import pytest

from bunker_amd import runtime as rt
from bunker_amd import synth

pytestmark = pytest.mark.gpu

bf = synth.f32_to_bf16
f32 = synth.bf16_to_f32


class Dev:
    def __init__(self):
        self.ptrs = []

    def up(self, a):
        p = rt.to_device(a); self.ptrs.append(p); return p

    def empty(self, nbytes):
        p = rt.cuAlloc(nbytes); rt.cuMemset(p, 0xCD, nbytes); self.ptrs.append(p); return p

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
    rc = rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], args)
    assert rc == 0, rt.last_error()
    rt.cuSync()


def ref_activation(orc, pro, x_bits, w_bits):
    """The Q8_1 rows the matmuls consume, per batch row."""
    rows = []
    for b in range(x_bits.shape[0]):
        h = orc.rmsnorm(x_bits[b], w_bits) if pro == 2 else x_bits[b]
        rows.append(orc.pack_q8_1(f32(h)))
    return rows


# K = 1024 / 2048 / 3584 / 4096 / 6144 run the fused kernel at batch < 8 (1024 and 3584 with lanes past the row in the last
# pass); K = 512 and batch 9 run the composed path
@pytest.mark.parametrize("K,batch,pro", [(2048, 1, 2), (2048, 3, 2), (2048, 1, 1), (2048, 2, 0), (4096, 1, 1), (6144, 2, 1),
                                          (6144, 1, 2), (512, 2, 2), (2048, 9, 2), (1024, 1, 2), (1024, 2, 0), (1024, 3, 1),
                                          (3584, 1, 1), (3584, 3, 2), (3584, 2, 0)])
def test_gemv_fused_groups(orc, dev, K, batch, pro):
    print(f"gemv_fused K={K} batch={batch} pro={pro}", flush=True)
    g = synth.rng(900 + K + 10 * batch + pro)
    Ns = [260, 130, 16, 18]            # not multiples of the rows a wave step covers
    epis = [1, 2, 0, 0]
    Ws = [synth.q4k_centered(g, n, K, 0.02) for n in Ns]
    x = bf(g.standard_normal((batch, K)).astype(np.float32))
    w = bf((g.standard_normal(K) * 0.1).astype(np.float32))
    res = bf(g.standard_normal((batch, Ns[1])).astype(np.float32))
    xq_rows = ref_activation(orc, pro, x, w)
    if pro == 0:
        dx = dev.up(np.stack(xq_rows))
    else:
        dx = dev.up(x)
    args = [dx] + ([dev.up(w)] if pro == 2 else [])
    outs = []
    for i, n in enumerate(Ns):
        args.append(dev.up(Ws[i]))
        if epis[i] == 2:
            args.append(dev.up(res))
        o = dev.empty(batch * n * (4 if epis[i] == 0 else 2)); outs.append(o); args.append(o)
    spec = f"gemv_fused K={K} pro={pro} G=4 batch={batch} " + " ".join(f"N{i}={n} epi{i}={e}" for i, (n, e) in enumerate(zip(Ns, epis)))
    launch(spec, args)
    for i, n in enumerate(Ns):
        for b in range(batch):
            y = orc.gemv_q4k_q8_1(Ws[i], xq_rows[b], n, K)
            if epis[i] == 0:
                got = rt.from_device(outs[i], (batch, n), np.float32)[b]
                assert np.array_equal(got.view(np.uint32), y.view(np.uint32)), (i, b)
            else:
                ref = orc.cast_bf16(y)
                if epis[i] == 2:
                    ref = orc.add_bf16(ref, res[b])
                got = rt.from_device(outs[i], (batch, n), np.uint16)[b]
                assert np.array_equal(got, ref), (i, b)


@pytest.mark.parametrize("K,N,batch", [(2048, 6144, 1), (2048, 204, 3), (512, 64, 2), (2048, 128, 8), (1024, 3584, 1), (1024, 100, 2),
                                       (768, 96, 70), (256, 64, 33), (6144, 32, 32)])
def test_gemv_fused_swiglu(orc, dev, K, N, batch):
    print(f"gemv_fused swiglu K={K} N={N} batch={batch}", flush=True)
    g = synth.rng(950 + N + batch)
    Wg, Wu = synth.q4k_centered(g, N, K, 0.05), synth.q4k_centered(g, N, K, 0.05)
    x = bf(g.standard_normal((batch, K)).astype(np.float32))
    w = bf((g.standard_normal(K) * 0.1).astype(np.float32))
    xq_rows = ref_activation(orc, 2, x, w)
    out = dev.empty(batch * N * 2)
    launch(f"gemv_fused K={K} pro=2 G=2 swiglu=1 N0={N} N1={N} batch={batch}", [dev.up(x), dev.up(w), dev.up(Wg), dev.up(Wu), out])
    got = rt.from_device(out, (batch, N), np.uint16)
    for b in range(batch):
        ref = orc.swiglu(orc.gemv_q4k_q8_1(Wg, xq_rows[b], N, K), orc.gemv_q4k_q8_1(Wu, xq_rows[b], N, K))
        assert np.array_equal(got[b], ref), b
    if batch >= 8 and N % 32 == 0:
        # the batched path can leave the activation as Q8_1 too (what the down projection would quantize itself)
        out2, q8 = dev.empty(batch * N * 2), dev.empty(batch * (N // 32) * 36)
        launch(f"gemv_fused K={K} pro=2 G=2 swiglu=1 N0={N} N1={N} batch={batch} q8out=1",
               [dev.up(x), dev.up(w), dev.up(Wg), dev.up(Wu), out2, q8])
        assert np.array_equal(rt.from_device(out2, (batch, N), np.uint16), got)
        gq = rt.from_device(q8, (batch, (N // 32) * 36), np.uint8)
        for b in range(batch):
            assert np.array_equal(gq[b], orc.pack_q8_1(f32(got[b]))), b
    elif batch < 8:
        with pytest.raises(rt.BunkerError, match="q8out"):
            rt.compileAndLoad(f"gemv_fused K=2048 pro=2 G=2 swiglu=1 N0=64 N1=64 batch={batch} q8out=1")


@pytest.mark.parametrize("Hg,B", [(16, 1), (3, 2)])
def test_gdn_conv_is_conv1d_then_delta_rule(orc, dev, Hg, B):
    """gdn_conv = conv1d_decode + gdn_delta_rule: output, S and the shifted conv state, to the bit."""
    print(f"gdn_conv Hg={Hg} B={B}", flush=True)
    g = synth.rng(700 + Hg + B)
    C = 3 * Hg * 128
    qkv = bf(g.standard_normal((B, C)).astype(np.float32))
    st = bf(g.standard_normal((B, 3, C)).astype(np.float32))
    cw = bf((g.standard_normal((C, 4)) * 0.5).astype(np.float32))
    z = bf(g.standard_normal((B, Hg * 128)).astype(np.float32))
    A_log = g.uniform(-2, 1, Hg).astype(np.float32)
    dt_bias = bf(g.standard_normal(Hg).astype(np.float32))
    a_p = g.standard_normal((B, Hg)).astype(np.float32); b_p = g.standard_normal((B, Hg)).astype(np.float32)
    norm_w = (1 + 0.1 * g.standard_normal(128)).astype(np.float32)
    S = (g.standard_normal((B, Hg, 128, 128)) * 0.02).astype(np.float32)
    dout, dS, dst = dev.empty(B * Hg * 128 * 2), dev.empty(S.nbytes), dev.up(st)
    dq8 = dev.empty(B * Hg * 4 * 36)
    launch(f"gdn_conv LVH={Hg} LKD=128 LVD=128 batch={B} q8out=1",
           [dev.up(qkv), dst, dev.up(cw), dev.up(z), dev.up(A_log), dev.up(dt_bias), dev.up(a_p), dev.up(b_p), dev.up(norm_w),
            dev.up(S), dout, dst, dS, dq8])        # conv state updated in place; the output also as Q8_1
    out = rt.from_device(dout, (B, Hg * 128), np.uint16); Sn = rt.from_device(dS, S.shape, np.float32)
    q8 = rt.from_device(dq8, (B, Hg * 4 * 36), np.uint8)
    for b in range(B):
        assert np.array_equal(q8[b], orc.pack_q8_1(f32(out[b]))), b
    stn = rt.from_device(dst, (B, 3, C), np.uint16)
    for b in range(B):
        conv, rs = orc.conv1d_decode(qkv[b], st[b], cw)
        ro, rS = orc.gdn_step(conv, z[b], A_log, dt_bias, a_p[b], b_p[b], norm_w, S[b], Hg, rows_per_chain=16)
        assert np.array_equal(stn[b], rs)
        assert np.array_equal(Sn[b].view(np.uint32), rS.view(np.uint32))
        assert np.array_equal(out[b], ro)


@pytest.mark.parametrize("batch", [1, 3])
def test_fa2_fused_is_norm_rope_append_attend(orc, dev, batch):
    """fa2_fused = qnorm, rope, knorm, ropek, cache append (all to the bit: the caches are compared) + attention
    (2e-2 max-abs against the checker fed with the same normalised, rotated q)."""
    print(f"fa2_fused batch={batch}", flush=True)
    g = synth.rng(720 + batch)
    NH, NKV, HD, HALF, MAXL = 16, 2, 256, 32, 512
    ppseq = MAXL // 16
    pos = [300, 15, 16][:batch]
    cos_t, sin_t = orc.rope_tables(MAXL, 64, 1e7)
    kc = bf(g.standard_normal((batch * ppseq, NKV, 16, HD)).astype(np.float32))
    vc = bf(g.standard_normal((batch * ppseq, NKV, 16, HD)).astype(np.float32))
    qgate = bf(g.standard_normal((batch, NH, 2, HD)).astype(np.float32))
    k = bf(g.standard_normal((batch, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((batch, NKV, HD)).astype(np.float32))
    qw = bf((g.standard_normal(HD) * 0.1).astype(np.float32)); kw = bf((g.standard_normal(HD) * 0.1).astype(np.float32))
    dkc, dvc = dev.up(kc), dev.up(rt.v_pages_to_device_layout(vc))
    dout = dev.empty(batch * NH * HD * 2)
    spec = f"fa2_fused HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} ROT_HALF={HALF}"
    common = [dev.up(qgate), dev.up(k), dev.up(v), dev.up(qw), dev.up(kw), dev.up(cos_t), dev.up(sin_t)]
    dq8 = dev.empty(batch * NH * HD // 32 * 36)
    if batch == 1:
        launch(spec + " q8out=1 splits=1", common + [pos[0], dkc, dvc, dout, dq8])        # one split: stand-alone quantizer
    else:
        launch(spec + f" batch={batch} pos_dev=1 q8out=1", common + [dev.up(np.array(pos, np.int32)), dkc, dvc, dout, dq8])
    out = rt.from_device(dout, (batch, NH, HD), np.uint16)
    q8 = rt.from_device(dq8, (batch, NH * HD // 32 * 36), np.uint8)
    for b in range(batch):
        assert np.array_equal(q8[b], orc.pack_q8_1(f32(out[b].ravel()))), b             # Q8_1 of the bf16 output as written
    bt = np.arange(batch * ppseq, dtype=np.int32).reshape(batch, ppseq)
    qn = np.empty((batch, NH, HD), np.uint16)
    for b in range(batch):
        qb = orc.headnorm(qgate[b].ravel(), qw, NH, HD, 2 * HD)
        qn[b] = orc.rope(qb, cos_t, sin_t, pos[b], NH, HD, HALF).reshape(NH, HD)
        kb = orc.rope(orc.headnorm(k[b].ravel(), kw, NKV, HD, HD), cos_t, sin_t, pos[b], NKV, HD, HALF)
        orc.kv_append(kb.reshape(NKV, HD), v[b], kc, vc, bt[b], pos[b], NKV, HD, 16)
    kc_d = rt.from_device(dkc, kc.shape, np.uint16)
    vc_d = rt.from_device(dvc, (batch * ppseq, NKV, HD, 16), np.uint16).transpose(0, 1, 3, 2)
    assert np.array_equal(kc_d, kc) and np.array_equal(vc_d, vc)
    ctx = np.array(pos, np.int32) + 1
    ro, _ = orc.attn_decode_paged(qn, kc, vc, bt, ctx, batch, NH, NKV, HD, 16, gate=qgate.ravel()[HD:],
                                  gate_bstride=NH * 2 * HD, gate_hstride=2 * HD)
    assert np.abs(f32(out).astype(np.float64) - f32(ro)).max() <= 2e-2


@pytest.mark.parametrize("batch", [8, 32])
def test_gemv_fused_short_matrices_inside_the_norm_launch(orc, dev, batch):
    """A batched projection group whose two large matrices alone fill the CUs with matmul tiles (6144 + 2048 rows = 256
    tiles) and whose two short ones (16 rows each) would add two more: the short ones are multiplied inside the
    RMSNorm -> Q8_1 launch.  Same bits as the checker's row loop for all four, and as the same op with the short
    matrices left in the matmul."""
    print(f"gemv_fused short matrices batch={batch}", flush=True)
    K, Ns, epis = 2048, [6144, 2048, 16, 16], [1, 1, 0, 0]
    g = synth.rng(4100 + batch)
    Ws = [synth.q4k_centered(g, n, K, 0.02) for n in Ns]
    x = bf(g.standard_normal((batch, K)).astype(np.float32))
    x[batch - 1] = 0                                         # an all-zero row: every Q8_1 scale is 0
    w = bf((g.standard_normal(K) * 0.1).astype(np.float32))
    xq_rows = ref_activation(orc, 2, x, w)
    spec = f"gemv_fused K={K} pro=2 G=4 batch={batch} " + " ".join(f"N{i}={n} epi{i}={e}" for i, (n, e) in enumerate(zip(Ns, epis)))
    got = {}
    try:
        for small in (1, 0):
            rt.tune_set("small_rows", small)
            args, outs = [dev.up(x), dev.up(w)], []
            for i, n in enumerate(Ns):
                o = dev.empty(batch * n * (4 if epis[i] == 0 else 2))
                rt.cuMemset(o, 0xff, batch * n * (4 if epis[i] == 0 else 2))
                outs.append(o); args += [dev.up(Ws[i]), o]
            launch(spec, args)
            got[small] = [rt.from_device(o, (batch, n), np.float32 if e == 0 else np.uint16) for o, n, e in zip(outs, Ns, epis)]
    finally:
        rt.tune_set("small_rows", 1)
    for i, n in enumerate(Ns):
        assert np.array_equal(got[1][i].view(np.uint32 if epis[i] == 0 else np.uint16), got[0][i].view(np.uint32 if epis[i] == 0 else np.uint16)), i
        for b in range(batch) if n <= 16 else (0, batch - 1):
            y = orc.gemv_q4k_q8_1(Ws[i], xq_rows[b], n, K)
            if epis[i] == 0:
                assert np.array_equal(got[1][i][b].view(np.uint32), y.view(np.uint32)), (i, b)
            else:
                assert np.array_equal(got[1][i][b], orc.cast_bf16(y)), (i, b)


@pytest.mark.parametrize("K,batch,C", [(2048, 1, 6144), (2048, 3, 390), (1024, 2, 6144), (1024, 1, 262)])
def test_gemv_fused_conv_epilogue_is_gemm_cast_conv1d(orc, dev, K, batch, C):
    """gemv_fused epi0=3: the rows of matrix 0 go through conv1d_decode in the kernel's last step (the slab form of a GDN
    layer).  Output, the shifted state (in place) and the other matrices of the group against the node sequence
    rmsnorm -> gemm (cast) -> conv1d_decode, to the bit; two steps in a row, the second on the state the first left.
    C = 390 / 262 are not multiples of the four rows of a wave step."""
    print(f"gemv_fused conv epilogue K={K} batch={batch} C={C}", flush=True)
    g = synth.rng(1300 + K + batch + C)
    Ns, epis = [C, 130, 16, 18], [3, 1, 0, 0]
    Ws = [synth.q4k_centered(g, n, K, 0.02) for n in Ns]
    w = bf((g.standard_normal(K) * 0.1).astype(np.float32))
    st = bf(g.standard_normal((batch, 3, C)).astype(np.float32))
    cw = bf((g.standard_normal((C, 4)) * 0.5).astype(np.float32))
    dst, dcw, dw = dev.up(st), dev.up(cw), dev.up(w)
    dWs = [dev.up(W) for W in Ws]
    outs = [dev.empty(batch * n * (4 if e == 0 else 2)) for n, e in zip(Ns, epis)]
    spec = f"gemv_fused K={K} pro=2 G=4 batch={batch} " + " ".join(f"N{i}={n} epi{i}={e}" for i, (n, e) in enumerate(zip(Ns, epis)))
    k = rt.compileAndLoad(spec)
    ref_st = [st[b] for b in range(batch)]
    for step in range(2):
        x = bf(g.standard_normal((batch, K)).astype(np.float32))
        args = [dev.up(x), dw, dWs[0], dst, dcw, outs[0], dst, dWs[1], outs[1], dWs[2], outs[2], dWs[3], outs[3]]
        assert rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], args) == 0, rt.last_error()
        rt.cuSync()
        xq_rows = ref_activation(orc, 2, x, w)
        got_conv = rt.from_device(outs[0], (batch, C), np.uint16)
        got_st = rt.from_device(dst, (batch, 3, C), np.uint16)
        for b in range(batch):
            qkv = orc.cast_bf16(orc.gemv_q4k_q8_1(Ws[0], xq_rows[b], C, K))
            conv, ref_st[b] = orc.conv1d_decode(qkv, ref_st[b], cw)
            assert np.array_equal(got_conv[b], conv), (step, b)
            assert np.array_equal(got_st[b], ref_st[b]), (step, b)
            assert np.array_equal(rt.from_device(outs[1], (batch, Ns[1]), np.uint16)[b], orc.cast_bf16(orc.gemv_q4k_q8_1(Ws[1], xq_rows[b], Ns[1], K)))
            for i in (2, 3):
                y = orc.gemv_q4k_q8_1(Ws[i], xq_rows[b], Ns[i], K)
                assert np.array_equal(rt.from_device(outs[i], (batch, Ns[i]), np.float32)[b].view(np.uint32), y.view(np.uint32))
    rt.unloadKernel(k)
    with pytest.raises(rt.BunkerError, match="epi"):
        rt.compileAndLoad("gemv_fused K=2048 pro=2 G=2 N0=64 epi0=1 N1=64 epi1=3")          # only matrix 0
    with pytest.raises(rt.BunkerError, match="epi"):
        rt.compileAndLoad("gemv_fused K=2048 pro=2 G=1 N0=64 epi0=3 batch=8")               # the batched path has no such step


@pytest.mark.parametrize("B", [1, 3])
def test_gdn_slabs_then_gated_norm_prologue_is_gdn_delta_rule_then_matmul(orc, dev, B):
    """gdn_slabs (four column slabs per head, raw outputs) followed by gemv_fused pro=3 (the gated RMS norm in the
    matmul's prologue) against gdn_delta_rule -> gemm -> cast -> add of the checker: state and the matmul's output to the
    bit, and the raw block's pieces against the checker's gated norm."""
    print(f"gdn_slabs + pro=3 B={B}", flush=True)
    g = synth.rng(1400 + B)
    Hg, H = 16, 520
    C = 3 * Hg * 128
    conv = bf(g.standard_normal((B, C)).astype(np.float32))
    z = bf(g.standard_normal((B, Hg * 128)).astype(np.float32))
    A_log = g.uniform(-2, 1, Hg).astype(np.float32)
    dt_bias = bf(g.standard_normal(Hg).astype(np.float32))
    a_p = g.standard_normal((B, Hg)).astype(np.float32); b_p = g.standard_normal((B, Hg)).astype(np.float32)
    norm_w = (1 + 0.1 * g.standard_normal(128)).astype(np.float32)
    S = (g.standard_normal((B, Hg, 128, 128)) * 0.02).astype(np.float32)
    Wo = synth.q4k_centered(g, H, Hg * 128, 0.02)
    res = bf(g.standard_normal((B, H)).astype(np.float32))
    raw_bytes = Hg * 128 * 8 + Hg * 32
    draw, dS, dnw = dev.empty(B * raw_bytes), dev.up(S), dev.up(norm_w)
    bp = f" batch={B}" if B != 1 else ""
    launch(f"gdn_slabs LVH={Hg} LKD=128 LVD=128" + bp,
           [dev.up(conv), dev.up(z), dev.up(A_log), dev.up(dt_bias), dev.up(a_p), dev.up(b_p), dS, draw, dS])      # S updated in place
    dout = dev.empty(B * H * 2)
    launch(f"gemv_fused K={Hg * 128} pro=3 G=1 N0={H} epi0=2" + bp, [draw, dnw, dev.up(Wo), dev.up(res), dout])
    Sn = rt.from_device(dS, S.shape, np.float32)
    out = rt.from_device(dout, (B, H), np.uint16)
    raw = rt.from_device(draw, (B, raw_bytes), np.uint8)
    for b in range(B):
        ro, rS = orc.gdn_step(conv[b], z[b], A_log, dt_bias, a_p[b], b_p[b], norm_w, S[b], Hg, rows_per_chain=16)
        assert np.array_equal(Sn[b].view(np.uint32), rS.view(np.uint32)), b
        y = orc.gemv_q4k_q8_1(Wo, orc.pack_q8_1(f32(ro)), H, Hg * 128)
        assert np.array_equal(out[b], orc.add_bf16(orc.cast_bf16(y), res[b])), b
        # the raw block: o and z * sigmoid(z) per column, the sum of o^2 per (head, slab)
        o = raw[b, :Hg * 128 * 4].view(np.float32).astype(np.float64).reshape(Hg, 4, 32)
        ss = raw[b, Hg * 128 * 8:].view(np.float64).reshape(Hg, 4)
        assert np.allclose(ss, (o ** 2).sum(axis=2), rtol=1e-14, atol=0)
    with pytest.raises(rt.BunkerError, match="pro=3"):
        rt.compileAndLoad("gemv_fused K=4096 pro=3 G=1 N0=64 epi0=2")
