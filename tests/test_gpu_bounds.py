"""Positions and lengths that live in device memory cannot be checked by a launcher, so the kernels hold them
inside the cache themselves: a cache write at a position outside 0..MAX_LEN-1 is skipped (the reference masks the same
store, src/emitters.ts:203-205), table reads use the nearest row, positions stop advancing at the capacity, and an
empty context gives zeros.  Every case here is laid out so that even an unclamped access would fall inside memory this
test allocated (spare pages and table rows behind the capacity, out-of-range rows never first in a buffer): the test
then fails on the comparison, not on the device."""
import numpy as np
import pytest

from bunker_amd import runtime as rt
from bunker_amd import synth

pytestmark = pytest.mark.gpu

bf = synth.f32_to_bf16
f32 = synth.bf16_to_f32
NH, NKV, HD, HALF = 16, 2, 256, 32


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
    rc = rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], args)
    assert rc == 0, rt.last_error()
    rt.cuSync()
    rt.unloadKernel(k)


def test_kv_append_writes_nothing_outside_the_cache(orc, dev):
    print("kv_append bounds", flush=True)
    g = synth.rng(901)
    B, MAXL, BT = 3, 32, 3                    # a sequence may hold 32 tokens; its block-table row has a spare third page
    pos = np.array([5, 32, -1], np.int32)     # inside; one past the capacity; negative (sequence 2: not first in the buffer)
    bt = np.arange(B * BT, dtype=np.int32).reshape(B, BT)
    kc = bf(g.standard_normal((B * BT, NKV, 16, HD)).astype(np.float32))
    vc = bf(g.standard_normal((B * BT, NKV, 16, HD)).astype(np.float32))
    k = bf(g.standard_normal((B, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((B, NKV, HD)).astype(np.float32))
    dkc, dvc = dev.up(kc), dev.up(rt.v_pages_to_device_layout(vc))
    rt.kv_append(dev.up(k), dev.up(v), dkc, dvc, dev.up(bt), BT, dev.up(pos), MAXL, B, NKV, HD, 16)
    rt.cuSync()
    orc.kv_append(k[0], v[0], kc, vc, bt[0], 5, NKV, HD, 16)            # only sequence 0's token lands
    kc_d = rt.from_device(dkc, kc.shape, np.uint16)
    vc_d = rt.from_device(dvc, (B * BT, NKV, HD, 16), np.uint16).transpose(0, 1, 3, 2)
    assert np.array_equal(kc_d, kc) and np.array_equal(vc_d, vc)
    # a capacity beyond the block-table row is refused on the host
    with pytest.raises(rt.BunkerError, match="exceeds the .* pages"):
        rt.kv_append(dev.up(k), dev.up(v), dkc, dvc, dev.up(bt), BT, dev.up(pos), 16 * BT + 1, B, NKV, HD, 16)


def test_fa2_fused_past_the_capacity_skips_the_append(orc, dev):
    """Sequence 1 arrives with pos == MAX_LEN (a loop replayed once too often): its K/V are not written, its rotation
    uses the table's last row, its query attends to the MAX_LEN tokens the cache holds.  Sequence 0 is unaffected."""
    print("fa2_fused bounds", flush=True)
    g = synth.rng(902)
    B, MAXL = 2, 32
    ppseq = MAXL // 16
    pos = np.array([7, MAXL], np.int32)
    cos_t, sin_t = orc.rope_tables(MAXL + 16, 64, 1e7)                   # spare rows behind the capacity
    npages = B * ppseq + 1                                               # one spare page behind the last sequence
    kc = bf(g.standard_normal((npages, NKV, 16, HD)).astype(np.float32))
    vc = bf(g.standard_normal((npages, NKV, 16, HD)).astype(np.float32))
    qgate = bf(g.standard_normal((B, NH, 2, HD)).astype(np.float32))
    k = bf(g.standard_normal((B, NKV, HD)).astype(np.float32)); v = bf(g.standard_normal((B, NKV, HD)).astype(np.float32))
    qw = bf((g.standard_normal(HD) * 0.1).astype(np.float32)); kw = bf((g.standard_normal(HD) * 0.1).astype(np.float32))
    dkc, dvc = dev.up(kc), dev.up(rt.v_pages_to_device_layout(vc))
    dout = dev.empty(B * NH * HD * 2)
    launch(f"fa2_fused HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} ROT_HALF={HALF} batch={B} pos_dev=1",
           [dev.up(qgate), dev.up(k), dev.up(v), dev.up(qw), dev.up(kw), dev.up(cos_t), dev.up(sin_t), dev.up(pos), dkc, dvc, dout])
    out = rt.from_device(dout, (B, NH, HD), np.uint16)
    bt = np.arange(B * ppseq, dtype=np.int32).reshape(B, ppseq)
    eff = [7, MAXL - 1]                                                  # the table row each sequence rotates with
    qn = np.empty((B, NH, HD), np.uint16)
    for b in range(B):
        qn[b] = orc.rope(orc.headnorm(qgate[b].ravel(), qw, NH, HD, 2 * HD), cos_t, sin_t, eff[b], NH, HD, HALF).reshape(NH, HD)
    kb = orc.rope(orc.headnorm(k[0].ravel(), kw, NKV, HD, HD), cos_t, sin_t, 7, NKV, HD, HALF)
    orc.kv_append(kb.reshape(NKV, HD), v[0], kc, vc, bt[0], 7, NKV, HD, 16)
    kc_d = rt.from_device(dkc, kc.shape, np.uint16)
    vc_d = rt.from_device(dvc, (npages, NKV, HD, 16), np.uint16).transpose(0, 1, 3, 2)
    assert np.array_equal(kc_d, kc) and np.array_equal(vc_d, vc)         # the spare page and sequence 1's pages untouched
    ctx = np.array([8, MAXL], np.int32)
    ro, _ = orc.attn_decode_paged(qn, kc, vc, bt, ctx, B, NH, NKV, HD, 16, gate=qgate.ravel()[HD:],
                                  gate_bstride=NH * 2 * HD, gate_hstride=2 * HD)
    assert np.abs(f32(out).astype(np.float64) - f32(ro)).max() <= 2e-2
    # a capacity that is not whole pages is refused when the handle is made
    with pytest.raises(rt.BunkerError, match="multiple of the 16-token page"):
        rt.compileAndLoad(f"fa2_fused HD={HD} NH={NH} NKV={NKV} MAX_LEN=40 ROT_HALF={HALF}")


def test_rope_reads_the_nearest_table_row(orc, dev):
    print("rope bounds", flush=True)
    g = synth.rng(903)
    B, MAXL = 3, 48
    cos_t, sin_t = orc.rope_tables(MAXL + 16, 64, 1e7)
    pos = np.array([47, 48, 60], np.int32)                               # last row; one past; well past (still inside the spare rows)
    x = bf(g.standard_normal((B, NH, HD)).astype(np.float32))
    dx = dev.up(x)
    launch(f"rope HD={HD} NH={NH} ROT_HALF={HALF} MAX_LEN={MAXL} batch={B} pos_dev=1", [dx, dev.up(cos_t), dev.up(sin_t), dev.up(pos)])
    got = rt.from_device(dx, (B, NH, HD), np.uint16)
    for b in range(B):
        assert np.array_equal(got[b].ravel(), orc.rope(x[b].ravel(), cos_t, sin_t, MAXL - 1, NH, HD, HALF)), b


def test_advance_stops_at_the_capacity(dev):
    print("advance bounds", flush=True)
    B = 2
    idx = np.array([11, 22], np.int32); val = np.array([1.5, -2.5], np.float32)
    dids, dpos = dev.up(np.zeros(B, np.int32)), dev.up(np.array([9, 3], np.int32))
    dhist, dcount = dev.up(np.zeros(4 * B * 2, np.int32)), dev.up(np.zeros(1, np.int32))
    k = rt.compileAndLoad(f"advance batch={B} max_steps=4 max_pos=10")
    for _ in range(3):
        assert rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], [dev.up(idx), dev.up(val), dids, dpos, dhist, dcount]) == 0, rt.last_error()
    rt.cuSync()
    assert rt.from_device(dpos, (B,), np.int32).tolist() == [10, 6]      # 9 -> 10 and no further; 3 -> 6
    assert rt.from_device(dids, (B,), np.int32).tolist() == [11, 22]
    assert rt.from_device(dcount, (1,), np.int32).tolist() == [3]
    with pytest.raises(rt.BunkerError, match="max_pos"):
        rt.compileAndLoad(f"advance batch={B} max_steps=4")
    # a destroyed handle refuses to launch
    rt.unloadKernel(k)
    assert rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], [dev.up(idx), dev.up(val), dids, dpos, dhist, dcount]) < 0
    assert "destroyed" in rt.last_error()


@pytest.mark.parametrize("splits", [1, 3])
def test_attention_lengths_outside_the_bound(orc, dev, splits):
    """ctx_len <= 0: zeros and lse = -inf; ctx_len > max_ctx: read as max_ctx, to the token (max_ctx = 60 ends inside a
    page).  The over-long length sits on a middle row, and every block-table row has four spare columns with valid page
    ids behind the four the bound allows (the caches hold those pages): a missing clamp would read memory of this test."""
    print(f"attn bounds splits={splits}", flush=True)
    g = synth.rng(904)
    B, L, L_alloc = 4, 60, 128
    kc, vc, bt, ctx = synth.paged_kv_random(g, B, L_alloc)          # 8 pages per table row, 32 pages in the caches
    ctx[:] = [40, 100, 0, 57]
    q = bf(g.standard_normal((B, NH, HD)).astype(np.float32))
    s, ws = rt.attn_plan(B, NKV, L, splits)
    assert s == splits
    dq, dkc, dvc, dbt, dctx = dev.up(q), dev.up(kc), dev.up(rt.v_pages_to_device_layout(vc)), dev.up(bt), dev.up(ctx)
    ref_ctx = np.array([40, 60, 1, 57], np.int32)
    ro, rl = orc.attn_decode_paged(q, kc, vc, bt, ref_ctx, B, NH, NKV, HD, 16)
    keep = [0, 1, 3]
    for exact in (False, True):
        if exact:
            s2, ws2 = rt.attn_plan_exact(B, NKV, L, splits)
        else:
            s2, ws2 = s, ws
        dws = dev.empty(ws2) if ws2 else 0
        dout, dlse = dev.empty(B * NH * HD * 2), dev.empty(B * NH * 4)
        (rt.attn_decode_exact if exact else rt.attn_decode)(dq, dkc, dvc, dbt, bt.shape[1], dctx, L, dout, dlse, B, NH, NKV, HD, 16, s2, dws, ws2)
        out = rt.from_device(dout, (B, NH, HD), np.uint16); lse = rt.from_device(dlse, (B, NH), np.float32)
        assert not out[2].any() and np.all(np.isneginf(lse[2])), exact
        if exact:
            assert np.array_equal(out[keep], ro[keep])
        assert np.abs(f32(out[keep]).astype(np.float64) - f32(ro[keep])).max() <= 2e-2, exact
        assert np.all(np.abs(lse[keep] - rl[keep]) <= 1e-4 * np.maximum(1, np.abs(rl[keep]))), exact
