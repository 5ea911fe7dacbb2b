"""Host logic without a GPU: the decode graph has the reference's shape (node count, op sequence,
slot order per op), the runner orders it correctly, and the CPU checker runs a tiny model."""
import numpy as np

from bunker_amd import model, runner, synth_model
from bunker_amd.model import REFERENCE, SYNTH, TINY


def test_node_count_and_op_sequence():
    g = model.buildModelGraph(SYNTH)
    # 1 + 18*17 + 6*19 + 3 (src/model.ts:46-204)
    assert len(g.nodes) == 424 == model.expected_node_count(SYNTH)
    assert len(model.buildModelGraph(REFERENCE).nodes) == 424
    ops = [n.op for n in g.nodes]
    gdn_layer = ["rmsnorm", "gemm", "gemm", "conv1d_decode", "gemm", "gemm", "gdn_delta_rule", "gemm", "cast", "add",
                 "rmsnorm", "gemm", "gemm", "swiglu", "gemm", "cast", "add"]
    fa_layer = ["rmsnorm", "gemm", "gemm", "gemm", "qnorm", "rope", "knorm", "ropek", "fa2_attn", "gemm", "cast", "add",
                "rmsnorm", "gemm", "gemm", "swiglu", "gemm", "cast", "add"]
    expect = ["embed"] + (gdn_layer * 3 + fa_layer) * 6 + ["rmsnorm", "gemm", "argmax"]
    assert ops == expect


def test_slot_order_per_op():
    g = model.buildModelGraph(SYNTH)
    plans = {p.group[0].op: p for p in runner.compilePartition(g, runner.choosePartition(g))}
    names = lambda op: [a.split("_", 1)[1] if a.startswith("n") and a[1].isdigit() else a for a in plans[op].args]
    assert names("embed") == ["embed.weight", "token_id", "out"]
    assert names("argmax") == ["out", "val", "idx"]
    assert [a.split(".")[-1] for a in names("fa2_attn")] == ["out", "out", "out", "out", "kv_k_in", "kv_v_in", "pos", "out",
                                                              "kv_k_new", "kv_v_new"]
    assert names("rope")[1:] == ["rope_cos", "rope_sin", "pos"] and len(plans["rope"].args) == 4
    gd = names("gdn_delta_rule")
    assert [a.split(".")[-1] for a in gd] == ["out", "out", "A_log", "dt_bias", "out", "out", "weight", "s_state_in", "out",
                                              "s_state_new"]
    cv = names("conv1d_decode")
    assert [a.split(".")[-1] for a in cv] == ["out", "conv_state_in", "weight", "out", "conv_state_new"]
    # residual adds: attention side is add(cast, h), MLP side is add(h, cast) (src/model.ts:113-117, 184-188)
    adds = [n for n in g.nodes if n.op == "add"]
    first, second = adds[0], adds[1]
    assert g.t(first.inputs[0].tensorName).producer.op == "cast"
    assert g.t(second.inputs[1].tensorName).producer.op == "cast"


def test_specs_carry_the_baked_constants():
    g = model.buildModelGraph(SYNTH, batch=4)
    specs = {n.op: runner.node_spec(n, 4, True) for n in g.nodes}
    assert specs["embed"] == "embed H=2048 VOCAB=151936 batch=4 ids_dev=1"
    assert specs["fa2_attn"] == "fa2_attn HD=256 NH=16 NKV=2 MAX_LEN=4352 batch=4 pos_dev=1"
    qkv = next(n for n in g.nodes if n.op == "gemm")
    assert runner.node_spec(qkv) == "gemm N=6144 K=2048 cast=1"


def test_topo_order_respects_dependencies_and_in_place_rope():
    g = model.buildModelGraph(TINY)
    # scramble the partition: the order must come from the dependencies alone
    part = runner.choosePartition(g)[::-1]
    order = [grp[0] for grp in runner.topoOrder(g, part)]
    posn = {n.id: i for i, n in enumerate(order)}
    for n in g.nodes:
        for d in g.deps()[n.id]:
            assert posn[d] < posn[n.id]
    for n in g.nodes:
        if n.op in ("rope", "ropek"):
            fa = next(c for c in g.t(n.inputs[0].tensorName).consumers if c.op == "fa2_attn")
            assert posn[n.id] < posn[fa.id]


def test_state_keys_and_bytes():
    assert runner.state_key("n12_model.layers.0.conv_state_new") == "model.layers.0.conv_state"
    assert runner.state_key("model.layers.3.kv_k_in") == "model.layers.3.kv_k"
    g = model.buildModelGraph(SYNTH)
    assert runner.tensor_bytes(g.t("lm_head.weight")) == 175030272
    assert runner.tensor_bytes(g.t("model.layers.0.s_state_in")) == 16 * 128 * 128 * 4
    total_q4k = sum(runner.tensor_bytes(t) for t in g.tensors.values() if t.type.dtype == "q4_k")
    assert 0.95e9 < total_q4k < 1.05e9          # ~990 MB of weights stream per token


def test_reference_model_runs_on_cpu(orc):
    from oracle.model_ref import RefModel
    W = synth_model.synth_weights(TINY, seed=5)
    S = synth_model.synth_state(TINY, batch=2, seed=6)
    m = RefModel(TINY, W, S, batch=2)
    toks, vals = m.decode([3, 700], [40, 41], steps=3)
    assert toks.shape == (3, 2) and toks.min() >= 0 and toks.max() < TINY.VOCAB
    m2 = RefModel(TINY, W, S, batch=2)
    t2, v2 = m2.decode([3, 700], [40, 41], steps=3)
    assert np.array_equal(toks, t2) and np.array_equal(vals, v2)
    # sequences are independent: sequence 1 alone gives the same tokens
    S1 = {k: v[1:2] for k, v in S.items()}
    t3, _ = RefModel(TINY, W, S1, batch=1).decode([700], [41], steps=3)
    assert np.array_equal(t3[:, 0], toks[:, 1])
    # the cache holds the new tokens' keys at positions 40..42 of sequence 0
    k0 = "model.layers.3.kv_k"
    assert not np.array_equal(m.S[k0][0, 40 // 16, :, 40 % 16], S[k0][0, 40 // 16, :, 40 % 16])
    assert np.array_equal(m.S[k0][0, 0], S[k0][0, 0])


def test_fused_partition_groups_and_specs():
    """Every node lands in exactly one group; the groups are the five fusions; a scrambled fused partition
    still orders by dependencies; the fused specs carry shapes and epilogues."""
    import collections
    g = model.buildModelGraph(SYNTH)
    part = runner.fusedPartition(g, slabs=False)
    ids = [n.id for grp in part for n in grp]
    assert sorted(ids) == [n.id for n in g.nodes]
    kinds = collections.Counter(tuple(n.op for n in grp) for grp in part)
    assert kinds[("rmsnorm", "gemm", "gemm", "gemm", "gemm")] == 18          # qkv, z, a, b
    assert kinds[("rmsnorm", "gemm", "gemm", "gemm")] == 6                   # q, k, v
    assert kinds[("rmsnorm", "gemm", "gemm", "swiglu")] == 24
    assert kinds[("gemm", "cast", "add")] == 48                             # out/o_proj and down with their residual adds
    assert kinds[("conv1d_decode", "gdn_delta_rule")] == 18
    assert kinds[("qnorm", "rope", "knorm", "ropek", "fa2_attn")] == 6
    assert kinds[("rmsnorm",)] == 1 and kinds[("gemm",)] == 1               # final norm and lm_head stay apart
    assert len(part) == 124
    ordered = runner.topoOrder(g, part[::-1])
    done = set()
    for grp in ordered:
        inside = {n.id for n in grp}
        for n in grp:
            for d in g.deps()[n.id]:
                assert d in done or d in inside
        done |= inside
    plans = runner.compilePartition(g, runner.topoOrder(g, part), 1, True)
    specs = [p.spec for p in plans]
    assert "gemv_fused K=2048 pro=2 G=4 N0=6144 epi0=1 N1=2048 epi1=1 N2=16 epi2=0 N3=16 epi3=0" in specs
    assert "gemv_fused K=2048 pro=2 G=2 swiglu=1 N0=6144 N1=6144" in specs
    assert "gemv_fused K=6144 pro=1 G=1 N0=2048 epi0=2" in specs
    assert "fa2_fused HD=256 NH=16 NKV=2 MAX_LEN=4352 ROT_HALF=32 pos_dev=1" in specs
    # At batch 1 (the default choice up to batch 7 for layers with ZD = 2048) a GDN layer is cut the other way: the
    # convolution joins the projections, the recurrence stands alone in its slab form and leaves raw outputs, and the
    # out_proj group reads those through its gated-norm prologue
    part_s = runner.fusedPartition(g)
    assert sorted(n.id for grp in part_s for n in grp) == [n.id for n in g.nodes] and len(part_s) == 124
    kinds_s = collections.Counter(tuple(sorted(n.op for n in grp)) for grp in part_s)
    assert kinds_s[("conv1d_decode", "gemm", "gemm", "gemm", "gemm", "rmsnorm")] == 18 and kinds_s[("gdn_delta_rule",)] == 18
    assert kinds_s[("conv1d_decode", "gdn_delta_rule")] == 0
    plans_s = runner.compilePartition(g, runner.topoOrder(g, part_s), 1, True)
    conv_plan = next(p for p in plans_s if "epi0=3" in p.spec)
    assert conv_plan.spec == "gemv_fused K=2048 pro=2 G=4 N0=6144 epi0=3 N1=2048 epi1=1 N2=16 epi2=0 N3=16 epi3=0" and len(conv_plan.args) == 13
    assert conv_plan.args[3] == "model.layers.0.conv_state_in" and conv_plan.args[6].endswith("conv_state_new")
    slab = next(p for p in plans_s if p.spec.startswith("gdn_slabs"))
    assert slab.spec == "gdn_slabs LVH=16 LKD=128 LVD=128" and list(slab.aux.values()) == [16 * 128 * 8 + 16 * 32]
    assert slab.args[0] == conv_plan.args[5] and slab.args[6] == "model.layers.0.s_state_in"
    outp = next(p for p in plans_s if p.args[0] == slab.args[7])
    assert outp.spec == "gemv_fused K=2048 pro=3 G=1 N0=2048 epi0=2" and outp.args[1] == "model.layers.0.linear_attn.norm.weight"
    assert sum(p.spec.startswith("gdn_slabs") for p in plans_s) == 18 and not any(p.spec.startswith("gdn_conv") for p in plans_s)
    # the small test model (ZD = 256) and batches from 8 on keep conv1d + recurrence in one launch
    gt = model.buildModelGraph(model.TINY)
    assert all(not p.spec.startswith("gdn_slabs") for p in runner.compilePartition(gt, runner.topoOrder(gt, runner.fusedPartition(gt)), 1, True))
    # from batch 8 on gdn_conv, fa2_fused and the SwiGLU group leave their output as Q8_1 too, and the projection behind
    # them reads that (pro=0) instead of quantizing
    g32 = model.buildModelGraph(SYNTH, 32)
    plans32 = runner.compilePartition(g32, runner.topoOrder(g32, runner.fusedPartition(g32)), 32, True)
    sw = next(p for p in plans32 if "swiglu=1" in p.spec)
    assert sw.spec == "gemv_fused K=2048 pro=2 G=2 swiglu=1 N0=6144 N1=6144 batch=32 q8out=1"
    assert list(sw.aux.values()) == [32 * (6144 // 32) * 36]
    down32 = next(p for p in plans32 if p.args[0] == sw.args[-1])
    assert down32.spec == "gemv_fused K=6144 pro=0 G=1 N0=2048 epi0=2 batch=32"
    gdn = next(p for p in plans32 if p.spec.startswith("gdn_conv"))
    assert gdn.spec.endswith("q8out=1") and list(gdn.aux.values()) == [32 * (2048 // 32) * 36]
    assert next(p for p in plans32 if p.args[0] == gdn.args[-1]).spec == "gemv_fused K=2048 pro=0 G=1 N0=2048 epi0=2 batch=32"
    fa = next(p for p in plans32 if p.spec.startswith("fa2_fused"))
    assert fa.spec.endswith("q8out=1")
    assert next(p for p in plans32 if p.args[0] == fa.args[-1]).spec == "gemv_fused K=4096 pro=0 G=1 N0=2048 epi0=2 batch=32"
    # lm_head reads the Q8_1 row the stand-alone final norm leaves in an auxiliary buffer
    norm = next(p for p in plans if p.spec.startswith("rmsnorm_q8_1"))
    head = next(p for p in plans if "N0=151936" in p.spec)
    assert list(norm.aux) == [head.args[0]] and "pro=0" in head.spec
    # residual of the fused matmul + cast + add is the add's other input
    down = next(p for p in plans if p.spec.startswith("gemv_fused K=6144"))
    assert g.t(down.args[2]).producer.op == "add" and g.t(down.args[3]).producer.op == "add"


class _NoDeviceEnv:
    """Stands in for a DecodeEnv in checks that must fail before anything touches the device."""
    inplace = True


def test_device_loop_refuses_runs_past_the_cache():
    """Positions advance on the device, so the capacity is checked on the host before any launch
    (the reference masks the same store, src/emitters.ts:203-205).  TINY holds 64 tokens."""
    import pytest

    from bunker_amd import model, runner

    gr = model.buildModelGraph(model.TINY, 2)
    assert runner.cache_capacity(gr) == model.TINY.MAX_LEN == 64
    env = _NoDeviceEnv()
    with pytest.raises(ValueError, match="exceeds the KV capacity"):
        runner.DeviceLoop(gr, env, 2, [1, 2], [10, 60], max_steps=5)        # 60 + 5 > 64
    with pytest.raises(ValueError, match="exceeds the KV capacity"):
        runner.DeviceLoop(gr, env, 2, [1, 2], 64, max_steps=1)
    with pytest.raises(ValueError, match="negative start position"):
        runner.DeviceLoop(gr, env, 2, [1, 2], [-1, 3], max_steps=2)
    with pytest.raises(ValueError, match="max_steps"):
        runner.DeviceLoop(gr, env, 2, [1, 2], 0, max_steps=0)
    # a run that fits passes the checks and only then needs the device
    try:
        runner.DeviceLoop(gr, env, 2, [1, 2], [10, 60], max_steps=4)
    except ValueError as e:       # pragma: no cover
        raise AssertionError(f"a run that fits was refused: {e}")
    except Exception:
        pass                      # no device here (or the stand-in env): anything but the capacity check


def test_dims_refuse_a_capacity_that_is_not_whole_pages():
    import pytest

    from bunker_amd import model

    with pytest.raises(ValueError, match="multiple of the 16-token page"):
        model.with_context(model.TINY, 100)
    with pytest.raises(ValueError, match="multiple of the 16-token page"):
        model.Dims(MAX_LEN=0)
    assert model.with_context(model.TINY, 128).MAX_LEN == 128
