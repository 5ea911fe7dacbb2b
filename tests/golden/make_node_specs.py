#!/usr/bin/env python3
"""Writes node_specs.json: the op spec string of every node and every fused group of the synthetic model's decode
graph, as the Python host layer (bunker_amd/runner.py, the code that runs against the GPU) builds them, for batch 1 and
batch 32 with token ids and positions in device memory.  tests/test_ts_specs.py expands the literal tables of
ts/specs.ts for the same nodes and groups and must get the same strings.

Needs no GPU and no built library (graph and partition code only).   Run:  python tests/golden/make_node_specs.py
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))

from bunker_amd import model, runner  # noqa: E402


def plans_of(D, batch, fused, attn_exact=True):
    g = model.buildModelGraph(D, batch)
    part = runner.fusedPartition(g) if fused else runner.choosePartition(g)
    ordered = runner.topoOrder(g, part)
    out = []
    for p in runner.compilePartition(g, ordered, batch, device_scalars=True, attn_exact=attn_exact):
        ops = [n.op for n in p.group]
        params = [{k: (int(v) if not isinstance(v, str) else v) for k, v in n.params.items()} for n in p.group]
        out.append({"ops": ops, "params": params, "spec": p.spec, "nargs": len(p.args), "aux_bytes": sorted(p.aux.values())})
    return out


def compact(plans):
    """Distinct plans once, plus the step's order as indices into them (layers repeat)."""
    table, index, order = [], {}, []
    for p in plans:
        key = json.dumps(p, sort_keys=True)
        if key not in index:
            index[key] = len(table)
            table.append(p)
        order.append(index[key])
    return {"distinct": table, "order": order}


def main():
    D = model.SYNTH
    doc = {"dims": {k: getattr(D, k) for k in ("H", "VOCAB", "NL", "FAI", "INTER", "NH", "NKV", "HD", "LKH", "LVH", "LKD", "LVD", "MAX_LEN", "ROT_DIM")},
           "device_scalars": True}
    for batch in (1, 32):
        doc[f"batch{batch}"] = {"nodes": compact(plans_of(D, batch, False)), "fused": compact(plans_of(D, batch, True))}
    doc["batch1_mfma_attention"] = {"fused": compact([p for p in plans_of(D, 1, True, attn_exact=False) if "fa2_attn" in p["ops"]]),
                                    "nodes": compact([p for p in plans_of(D, 1, False, attn_exact=False) if "fa2_attn" in p["ops"]])}
    with open(os.path.join(HERE, "node_specs.json"), "w") as f:
        json.dump(doc, f, separators=(",", ":"))
        f.write("\n")
    print({k: (len(v["nodes"]["order"]), len(v["fused"]["order"])) for k, v in doc.items() if isinstance(v, dict) and "nodes" in v})


if __name__ == "__main__":
    main()
