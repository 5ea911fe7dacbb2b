"""bk_attn_decode_noalloc — the split-K decode attention for callers that cannot allocate — against bk_attn_decode
with a caller's workspace: same bits for the same number of splits, on two calls in a row that share the library's
fixed scratch array, the second with a smaller input (whose partials land on the first call's leftovers); the small
call also against the CPU checker (2e-2 max-abs on the bf16 output, 1e-4 relative on the log-sum-exp)."""
import numpy as np
import pytest

from bunker_amd import runtime as rt
from bunker_amd import synth

pytestmark = pytest.mark.gpu

bf = synth.f32_to_bf16
f32 = synth.bf16_to_f32
NH, NKV, HD = 16, 2, 256


def _both(g, B, L, splits_req=0, own_choice=False):
    """One problem through both entry points; returns (out, lse) of each and the inputs.  own_choice: the no-alloc
    entry point is handed splits = 0 and picks the count itself, the workspace form gets what bk_attn_plan returns."""
    kc, vc, bt, ctx = synth.paged_kv_random(g, B, L)
    q = bf(g.standard_normal((B, NH, HD)).astype(np.float32))
    splits, ws = rt.attn_plan(B, NKV, L, splits_req)
    ptrs = []

    def up(a):
        p = rt.to_device(a); ptrs.append(p); return p

    def empty(n):
        p = rt.cuAlloc(n); ptrs.append(p); return p

    dq, dkc, dvc, dbt, dctx = up(q), up(kc), up(rt.v_pages_to_device_layout(vc)), up(bt), up(ctx)
    dws = empty(ws) if ws else 0
    o1, l1, o2, l2 = empty(B * NH * HD * 2), empty(B * NH * 4), empty(B * NH * HD * 2), empty(B * NH * 4)
    for p in (o1, o2):
        rt.cuMemset(p, 0xFF, B * NH * HD * 2)
    print(f"attn_decode_noalloc B={B} L={L} splits={splits}", flush=True)
    rt.attn_decode_noalloc(dq, dkc, dvc, dbt, bt.shape[1], dctx, L, o1, l1, B, NH, NKV, HD, 16, 0 if own_choice else splits)
    rt.attn_decode(dq, dkc, dvc, dbt, bt.shape[1], dctx, L, o2, l2, B, NH, NKV, HD, 16, splits, dws, ws)
    rt.cuSync()
    res = (rt.from_device(o1, (B, NH, HD), np.uint16), rt.from_device(l1, (B, NH), np.float32),
           rt.from_device(o2, (B, NH, HD), np.uint16), rt.from_device(l2, (B, NH), np.float32))
    for p in ptrs:
        rt.cuFree(p)
    return res, (q, kc, vc, bt, ctx), splits


def test_noalloc_attention_equals_the_workspace_form(orc):
    g = synth.rng(950)
    # first call: long contexts, many splits (the balanced plan: 8 x 16 slots)
    (o1, l1, o2, l2), _, s_big = _both(g, 8, 16384)
    assert s_big > 1
    assert np.array_equal(o1, o2) and np.array_equal(l1.view(np.uint32), l2.view(np.uint32))
    # second call: smaller batch, shorter contexts, fewer partials, on the same array
    (o1, l1, o2, l2), (q, kc, vc, bt, ctx), s_small = _both(g, 2, 1000)
    assert 1 < s_small
    assert np.array_equal(o1, o2) and np.array_equal(l1.view(np.uint32), l2.view(np.uint32))
    ro, rl = orc.attn_decode_paged(q, kc, vc, bt, ctx, 2, NH, NKV, HD, 16)
    assert np.abs(f32(o1).astype(np.float64) - f32(ro)).max() <= 2e-2
    assert np.all(np.abs(l1 - rl) <= 1e-4 * np.maximum(1, np.abs(rl)))
    # a third: the no-alloc entry point itself is handed splits = 0 (its own choice, held to what the array takes) and
    # must cut the pages like bk_attn_decode at the count bk_attn_plan returns; also against the checker
    (o1, l1, o2, l2), (q, kc, vc, bt, ctx), s_own = _both(g, 3, 4096, 0, own_choice=True)
    assert s_own > 1
    assert np.array_equal(o1, o2) and np.array_equal(l1.view(np.uint32), l2.view(np.uint32))
    ro, rl = orc.attn_decode_paged(q, kc, vc, bt, ctx, 3, NH, NKV, HD, 16)
    assert np.abs(f32(o1).astype(np.float64) - f32(ro)).max() <= 2e-2
    assert np.all(np.abs(l1 - rl) <= 1e-4 * np.maximum(1, np.abs(rl)))


def test_noalloc_attention_refuses_more_partials_than_the_array_holds():
    """batch * NKV * splits beyond 1024 is an error before anything is launched (the pointers are never used)."""
    p = rt.cuAlloc(4096)
    try:
        with pytest.raises(rt.BunkerError, match="exceed the 1024 of the built-in scratch"):
            rt.attn_decode_noalloc(p, p, p, 0, 1024, p, 16384, p, 0, 64, NH, NKV, HD, 16, splits=16)
    finally:
        rt.cuFree(p)
