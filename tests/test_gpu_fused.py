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


# K = 2048 / 4096 / 6144 run the fused kernel at batch < 8; K = 512 and batch 9 run the composed path
@pytest.mark.parametrize("K,batch,pro", [(2048, 1, 2), (2048, 3, 2), (2048, 1, 1), (2048, 2, 0), (4096, 1, 1), (6144, 2, 1),
                                          (6144, 1, 2), (512, 2, 2), (2048, 9, 2)])
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


@pytest.mark.parametrize("K,N,batch", [(2048, 6144, 1), (2048, 204, 3), (512, 64, 2), (2048, 128, 8)])
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
