"""ts/specs.ts against the Python host layer, as text (bun cannot run here).

The TypeScript glue a maintainer drops next to src/runner.ts builds its op spec strings from three literal tables
(SPEC_KEYS, FUSED_SPECS, SPEC_SUFFIX).  This test reads those tables out of the file, expands them with plain ${name}
substitution — the only thing `fill` in specs.ts does — for every node (424) and every fused group (124 plans) of the
synthetic model at batch 1 and 32, and compares with tests/golden/node_specs.json, which tests/golden/make_node_specs.py
writes from bunker_amd/runner.py (the code the GPU tests run).  It also checks that the fixture is what the host layer
produces today, and the constants and exports the call sites need."""
import json
import os
import re

import pytest

from bunker_amd import model, runner

ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
TS = open(os.path.join(ROOT, "ts", "specs.ts")).read()
GOLD = json.load(open(os.path.join(ROOT, "tests", "golden", "node_specs.json")))


def ts_table(name):
    """The body of `export const <name>: Record<...> = { ... };` as a dict (string -> string, or string -> list of strings)."""
    m = re.search(r"export const %s: Record<[^>]+> = \{(.*?)\n\};" % name, TS, flags=re.S)
    assert m, name
    out = {}
    for key, val in re.findall(r'^\s*"([^"]+)":\s*(\[[^\]]*\]|"[^"]*"),', m.group(1), flags=re.M):
        out[key] = re.findall(r'"([^"]*)"', val) if val.startswith("[") else val[1:-1]
    return out


def ts_const(name):
    return int(re.search(r"export const %s = (\d+);" % name, TS).group(1))


SPEC_KEYS, FUSED, SUFFIX = ts_table("SPEC_KEYS"), ts_table("FUSED_SPECS"), ts_table("SPEC_SUFFIX")


def fill(template, **v):
    return re.sub(r"\$\{(\w+)\}", lambda m: str(v[m.group(1)]), template)


def expand(plan, batch, attn_exact, q8_in):
    """What nodeSpec / groupPlan / compilePartition of specs.ts return for this plan, using only the file's tables."""
    ops, P = plan["ops"], plan["params"]
    key = "+".join(ops)
    bpart = fill(SUFFIX["batch"], batch=batch) if batch != 1 else ""
    q8out = SUFFIX["q8out"] if batch >= ts_const("Q8OUT_MIN_BATCH") else ""
    if len(ops) == 1:
        op, p = ops[0], P[0]
        if plan["spec"].startswith("gdn_slabs"):
            return fill(FUSED["gdn_slabs"], LVH=p["LVH"], LKD=p["LKD"], LVD=p["LVD"]) + bpart
        if plan["spec"].startswith("rmsnorm_q8_1"):
            return fill(FUSED["rmsnorm_q8_1"], N=p["N"]) + bpart
        if op == "gemm" and q8_in:
            return fill(FUSED["gemm@q8_1"], K=p["K"], N=p["N"], EPI=1 if p.get("cast") else 0) + bpart
        s = " ".join([op] + [f"{k}={p[k]}" for k in SPEC_KEYS[op]])
        if op == "gemm" and p.get("cast"):
            s += SUFFIX["cast"]
        s += bpart
        if op == "embed":
            s += SUFFIX["ids_dev"]
        if op in ("rope", "ropek", "fa2_attn"):
            s += SUFFIX["pos_dev"]
        if op == "fa2_attn" and not attn_exact:
            s += SUFFIX["exact0"]
        return s
    if key == "rmsnorm+gemm+gemm+swiglu":
        return fill(FUSED[key], K=P[1]["K"], N=P[1]["N"]) + bpart + (q8out if P[1]["N"] % 32 == 0 else "")
    if ops[0] == "rmsnorm" and "conv1d_decode" in ops:
        gem = [p for o, p in zip(ops, P) if o == "gemm"]
        mats = "".join(fill(FUSED["mat"], i=i, N=p["N"], EPI=3 if i == 0 else (1 if p.get("cast") else 0)) for i, p in enumerate(gem))
        return fill(FUSED["rmsnorm+gemm*+conv1d_decode"], K=gem[0]["K"], MATS=mats) + bpart
    if ops[0] == "rmsnorm" and all(o == "gemm" for o in ops[1:]):
        mats = "".join(fill(FUSED["mat"], i=i, N=p["N"], EPI=1 if p.get("cast") else 0) for i, p in enumerate(P[1:]))
        return fill(FUSED["rmsnorm+gemm*"], K=P[1]["K"], G=len(ops) - 1, MATS=mats) + bpart
    if key == "gemm+cast+add":
        if " pro=3 " in plan["spec"]:        # reads the raw block of a gdn_slabs op (rawOf in specs.ts)
            return fill(FUSED["gemm+cast+add@raw"], K=P[0]["K"], N=P[0]["N"]) + bpart
        return fill(FUSED[key], K=P[0]["K"], N=P[0]["N"], PRO=0 if q8_in else 1) + bpart
    if key == "conv1d_decode+gdn_delta_rule":
        return fill(FUSED[key], LVH=P[1]["LVH"], LKD=P[1]["LKD"], LVD=P[1]["LVD"]) + bpart + q8out
    if key == "qnorm+rope+knorm+ropek+fa2_attn":
        fa, rp = P[4], P[1]
        return fill(FUSED[key], HD=fa["HD"], NH=fa["NH"], NKV=fa["NKV"], MAX_LEN=fa["MAX_LEN"], ROT_HALF=rp["ROT_HALF"]) + bpart + \
            SUFFIX["pos_dev"] + ("" if attn_exact else SUFFIX["exact0"]) + q8out
    raise AssertionError(key)


@pytest.mark.parametrize("section,batch,attn_exact", [("batch1", 1, True), ("batch32", 32, True), ("batch1_mfma_attention", 1, False)])
def test_ts_tables_expand_to_the_host_layers_specs(section, batch, attn_exact):
    for kind in ("nodes", "fused"):
        table = GOLD[section][kind]
        plans = [table["distinct"][i] for i in table["order"]]
        if section in ("batch1", "batch32"):
            assert len(plans) == (424 if kind == "nodes" else 124)
        for p in plans:
            # whether the activation the matmul reads already exists as Q8_1 is the partition's bookkeeping (q8Of in
            # specs.ts); the fixture shows it in the spec it recorded
            q8_in = " pro=0 " in p["spec"]
            assert expand(p, batch, attn_exact, q8_in) == p["spec"], (kind, p["ops"])


def test_fixture_is_what_the_host_layer_builds_today():
    D = model.SYNTH
    assert {k: getattr(D, k) for k in GOLD["dims"]} == GOLD["dims"]
    for batch in (1, 32):
        g = model.buildModelGraph(D, batch)
        for kind, part in (("nodes", runner.choosePartition(g)), ("fused", runner.fusedPartition(g))):
            plans = runner.compilePartition(g, runner.topoOrder(g, part), batch, device_scalars=True)
            table = GOLD[f"batch{batch}"][kind]
            gold = [table["distinct"][i] for i in table["order"]]
            assert [p.spec for p in plans] == [p["spec"] for p in gold]
            assert [len(p.args) for p in plans] == [p["nargs"] for p in gold]
            assert [sorted(p.aux.values()) for p in plans] == [p["aux_bytes"] for p in gold]


def test_ts_constants_and_exports():
    assert SPEC_KEYS == runner._SPEC_KEYS                      # the same 14 ops, the same constants in the same order
    assert ts_const("Q8OUT_MIN_BATCH") == runner.Q8OUT_MIN_BATCH and ts_const("LM_HEAD_ROWS") == runner.LM_HEAD_ROWS
    assert ts_const("SLAB_MAX_BATCH") == runner.SLAB_MAX_BATCH
    assert ts_const("PAGE_TOKENS") == 16
    for fn in ("nodeSpec", "groupPlan", "compilePartition", "loadPartition", "stateBytes", "ropeTables"):
        assert re.search(r"^export function %s\(" % fn, TS, flags=re.M), fn
    # every fused group the Python partition forms has a template, and the templates name only variables groupPlan fills
    keys = {"+".join(p["ops"]) for b in ("batch1", "batch32") for p in GOLD[b]["fused"]["distinct"] if len(p["ops"]) > 1}
    for k in keys:
        assert k in FUSED or (k.startswith("rmsnorm+gemm") and ("rmsnorm+gemm*+conv1d_decode" if "conv1d_decode" in k else "rmsnorm+gemm*") in FUSED), k
    # state sizes of stateBytes are the graph's tensor sizes
    D, B = model.SYNTH, 3
    g = model.buildModelGraph(D, B)
    sizes = {"conv_state": B * 3 * D.QKVD * 2, "s_state": B * D.LVH * D.LKD * D.LVD * 4, "kv_k": B * D.NKV * D.MAX_LEN * D.HD * 2}
    assert runner.tensor_bytes(g.t("model.layers.0.conv_state_in")) == sizes["conv_state"]
    assert runner.tensor_bytes(g.t("model.layers.0.s_state_in")) == sizes["s_state"]
    assert runner.tensor_bytes(g.t("model.layers.3.kv_k_in")) == sizes["kv_k"]
    for expr in ("batch * 3 * QKVD * 2", "batch * D.LVH * D.LKD * D.LVD * 4", "batch * D.NKV * D.MAX_LEN * D.HD * 2"):
        assert expr in TS, expr
