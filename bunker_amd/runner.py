"""Graph-driven decode runtime: partition -> topological order -> kernels -> token loop.

Counterpart of src/runner.ts (``choosePartition``, ``topoOrder``, ``compileStep``,
``runGraphDecode``) and of the buffer plumbing of prototypes/decode_graph.ts:66-145
(``DecodeEnv``: state double buffers, rope tables, scratch for intermediates).  Each
group of the partition becomes one pre-compiled kernel handle (``compileAndLoad`` of an op
spec instead of TTIR text) and one ``cuLaunch`` per token with the node's tensors in the
reference's slot order: inputs in declared order, then outputs (src/fusion.ts:371-401).

``runGraphDecode`` is the reference's loop: token id and position are passed as scalars and
every kernel is launched from the host each step.  ``DeviceLoop`` is the fast path of this
build: token ids and positions live in device memory, one step is recorded once into a HIP
graph and replayed, and the generated tokens are read back at the end.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable

import numpy as np

from . import runtime as rt
from . import synth
from .graph import Graph, GraphNode
from .model import Dims, SYNTH, buildModelGraph

Partition = list  # list[list[GraphNode]]


@dataclass
class KernelPlan:
    """What compilePartition returns per group (src/fusion.ts:110-117), with an op spec for ttir."""
    spec: str
    name: str
    args: list            # external tensor names, in slot order
    grid: list
    group: list
    aux: dict = field(default_factory=dict)   # name -> bytes of buffers that exist only between fused kernels


@dataclass
class CompiledStep:
    graph: Graph
    schedule: list        # [(KernelPlan, LoadedKernel)]
    batch: int = 1
    device_scalars: bool = False


# ---------------------------------------------------------------- partition + order
def choosePartition(graph: Graph, env=None, opts: dict | None = None) -> Partition:
    """Every node its own kernel (src/runner.ts:40-49)."""
    return [[n] for n in graph.nodes]


LM_HEAD_ROWS = 32768     # matmuls with more rows keep the stand-alone norm + quantizer (its cost is paid once, not per workgroup)


SLAB_MAX_BATCH = 7       # up to this batch the GDN step runs in column slabs (64 workgroups for 16 heads instead of 16)


def graph_batch(graph: Graph) -> int:
    """Sequences per step of a graph built by buildModelGraph (the leading dimension of its activations)."""
    return int(graph.nodes[0].outputs[0].type.shape[0])


def gdn_slab_form(gd: GraphNode, proj_K: int, batch: int) -> bool:
    """Whether a GDN layer runs as [norm + projections + conv1d] [gdn_slabs] [gated norm + out_proj + add]: the kernels
    exist for heads of 128 x 128, ZD = 2048 and projection rows of 1024 or 2048 at batch < 8."""
    return (batch <= SLAB_MAX_BATCH and int(gd.params["ZD"]) == 2048 and int(gd.params["LKD"]) == 128 and int(gd.params["LVD"]) == 128
            and proj_K in (1024, 2048))


def fusedPartition(graph: Graph, slabs: bool | None = None) -> Partition:
    """Groups of nodes that one fused kernel (or one short kernel sequence) serves.

    The counterpart of src/fusion.ts's partitioning, with the fusions that pay on this hardware:
      rmsnorm + the matmuls that read it                      (norm and Q8_1 in the GEMV prologue)
      rmsnorm + gate + up + swiglu                            (SwiGLU in the GEMV epilogue)
      matmul + cast + add                                     (residual add in the GEMV epilogue)
      conv1d_decode + gdn_delta_rule                          (the conv output stays on chip)
      qnorm + rope + knorm + ropek + fa2_attn                 (norm, rotation and cache append in one launch)
    A group is formed only when no tensor produced inside it (other than its declared result) is read outside.
    At small batch (``slabs``; None = decided from the graph by gdn_slab_form) a GDN layer is cut differently, so that
    its recurrence can run in column slabs on four times as many CUs: conv1d_decode joins the projections in front of it
    (the convolution is the last step of the qkv rows), gdn_delta_rule stands alone and leaves its gated norm to the
    out_proj group behind it (compilePartition: gdn_slabs, gemv_fused pro=3).
    """
    taken: set = set()
    groups: dict[int, list] = {}          # first node id -> group
    batch = graph_batch(graph)

    def consumers(t):
        return graph.tensors[t].consumers

    def only_inside(nodes, results):
        ids = {n.id for n in nodes}
        for n in nodes:
            for o in n.outputs:
                if o.tensorName in results or graph.tensors[o.tensorName].role == "state":
                    continue
                if any(c.id not in ids for c in consumers(o.tensorName)):
                    return False
        return True

    def take(nodes):
        nodes = sorted(nodes, key=lambda n: n.id)
        groups[nodes[0].id] = nodes
        taken.update(n.id for n in nodes)

    for n in graph.nodes:
        if n.id in taken:
            continue
        if n.op == "rmsnorm":
            cons = consumers(n.outputs[0].tensorName)
            if cons and all(c.op == "gemm" and c.inputs[0].tensorName == n.outputs[0].tensorName for c in cons) and len(cons) <= 4:
                if max(int(c.params["N"]) for c in cons) > LM_HEAD_ROWS:
                    continue
                sw = None
                if len(cons) == 2:
                    c0, c1 = (consumers(c.outputs[0].tensorName) for c in cons)
                    if len(c0) == 1 and len(c1) == 1 and c0[0] is c1[0] and c0[0].op == "swiglu" and not cons[0].params.get("cast") \
                            and int(cons[0].params["N"]) % 4 == 0:
                        sw = c0[0]
                nodes = [n] + list(cons) + ([sw] if sw else [])
                results = {sw.outputs[0].tensorName} if sw else {c.outputs[0].tensorName for c in cons}
                # slab form of a GDN layer: the convolution that reads the first matmul's rows joins the group
                cv = consumers(cons[0].outputs[0].tensorName)
                if not sw and len(cons) == 4 and len(cv) == 1 and cv[0].op == "conv1d_decode" and cons[0].params.get("cast"):
                    gd = consumers(cv[0].outputs[0].tensorName)
                    use = slabs if slabs is not None else (len(gd) == 1 and gd[0].op == "gdn_delta_rule" and
                                                          gdn_slab_form(gd[0], int(cons[0].params["K"]), batch))
                    if use and len(gd) == 1 and gd[0].op == "gdn_delta_rule":
                        nodes.append(cv[0])
                        results = (results - {cons[0].outputs[0].tensorName}) | {cv[0].outputs[0].tensorName}
                if only_inside(nodes, results):
                    take(nodes)
        elif n.op == "gemm" and not n.params.get("cast"):
            c = consumers(n.outputs[0].tensorName)
            if len(c) == 1 and c[0].op == "cast":
                a = consumers(c[0].outputs[0].tensorName)
                if len(a) == 1 and a[0].op == "add" and a[0].id not in taken:
                    take([n, c[0], a[0]])
        elif n.op == "conv1d_decode":
            c = consumers(n.outputs[0].tensorName)
            if len(c) == 1 and c[0].op == "gdn_delta_rule" and c[0].inputs[0].tensorName == n.outputs[0].tensorName:
                take([n, c[0]])
        elif n.op == "qnorm":
            qn_out = n.outputs[0].tensorName
            fa = next((c for c in consumers(qn_out) if c.op == "fa2_attn"), None)
            rope = next((c for c in consumers(qn_out) if c.op == "rope"), None)
            if fa is None or rope is None:
                continue
            kn = graph.tensors[fa.inputs[1].tensorName].producer
            ropek = next((c for c in consumers(kn.outputs[0].tensorName) if c.op == "ropek"), None) if kn is not None and kn.op == "knorm" else None
            if ropek is None or fa.inputs[3].tensorName != n.inputs[0].tensorName:
                continue
            nodes = [n, rope, kn, ropek, fa]
            if only_inside(nodes, {fa.outputs[0].tensorName}):
                take(nodes)
    out = []
    for n in graph.nodes:
        if n.id in groups:
            out.append(groups[n.id])
        elif n.id not in taken:
            out.append([n])
    return out


def topoOrder(graph: Graph, partition: Partition) -> Partition:
    """Kahn's algorithm over groups with a FIFO queue (src/runner.ts:52-91).

    One rule is added: a node without outputs that rewrites its first input in place (rope,
    ropek) must run before the later consumers of that tensor.  The reference gets that order
    only from queue order (src/runner.ts:69-88); here it is an edge of its own.
    """
    node_group = {}
    for gi, grp in enumerate(partition):
        for n in grp:
            node_group[n.id] = gi
    edges: dict[int, list] = {gi: [] for gi in range(len(partition))}
    indeg = {gi: 0 for gi in range(len(partition))}

    def add_edge(a, b):
        if a != b:
            edges[a].append(b)
            indeg[b] += 1

    for gi, grp in enumerate(partition):
        for n in grp:
            for inp in n.inputs:
                p = graph.tensors[inp.tensorName].producer
                if p is not None:
                    add_edge(node_group[p.id], gi)
    for n in graph.nodes:
        if not n.outputs and n.inputs:
            t = graph.tensors[n.inputs[0].tensorName]
            for c in t.consumers:
                if c.id > n.id:
                    add_edge(node_group[n.id], node_group[c.id])
    queue = [gi for gi in range(len(partition)) if indeg[gi] == 0]
    out = []
    while queue:
        gi = queue.pop(0)
        out.append(partition[gi])
        for b in edges[gi]:
            indeg[b] -= 1
            if indeg[b] == 0:
                queue.append(b)
    if len(out) != len(partition):
        raise RuntimeError(f"topoOrder: cycle in partition ({len(out)}/{len(partition)})")
    return out


_SPEC_KEYS = {
    "embed": ["H", "VOCAB"], "rmsnorm": ["N"], "gemm": ["N", "K"], "cast": ["N"], "add": ["N"], "swiglu": ["N"],
    "conv1d_decode": ["QKVD"], "gdn_delta_rule": ["LVH", "LKD", "LVD"], "qnorm": ["HD", "NH"], "knorm": ["HD", "NKV"],
    "rope": ["HD", "NH", "ROT_HALF", "MAX_LEN"], "ropek": ["HD", "NKV", "ROT_HALF", "MAX_LEN"],
    "fa2_attn": ["HD", "NH", "NKV", "MAX_LEN"], "argmax": ["VOCAB"],
}


def node_spec(n: GraphNode, batch: int = 1, device_scalars: bool = False, attn_exact: bool = True) -> str:
    """Op name plus the constants the reference baked into the kernel text."""
    parts = [n.op] + [f"{k}={int(n.params[k])}" for k in _SPEC_KEYS[n.op]]
    if n.op == "gemm" and n.params.get("cast"):
        parts.append("cast=1")
    if batch != 1:
        parts.append(f"batch={batch}")
    if device_scalars:
        if n.op == "embed":
            parts.append("ids_dev=1")
        if n.op in ("rope", "ropek", "fa2_attn"):
            parts.append("pos_dev=1")
    if n.op == "fa2_attn" and not attn_exact:
        parts.append("exact=0")
    return " ".join(parts)


# attn_exact (an argument of node_spec, compilePartition, compileStep, DeviceLoop and prefill.Prefill): attention ops
# run their double-precision form by default (the checker's bits, so a decode reproduces the host evaluation token for
# token); False selects the bf16 matrix-instruction form (within 2e-2, 1.5 to 1.8 times faster on the attention
# launches themselves) for the plans of that call only.

Q8OUT_MIN_BATCH = 8      # from this batch on producers also emit their output as Q8_1 (gemv_fused then runs its batched path)


def _group_plan(graph: Graph, grp: list, batch: int, device_scalars: bool, q8_of: dict, attn_exact: bool = True,
                raw_of: dict | None = None) -> KernelPlan:
    """The fused op spec and slot list for a multi-node group (see fusedPartition)."""
    ops = tuple(n.op for n in grp)
    bpart = f" batch={batch}" if batch != 1 else ""
    name = "+".join(ops) + f"_{grp[0].id}"
    raw_of = raw_of if raw_of is not None else {}
    if ops[0] == "rmsnorm" and sorted(ops[1:]) == ["conv1d_decode", "gemm", "gemm", "gemm", "gemm"]:
        norm, gemms, cv = grp[0], [n for n in grp if n.op == "gemm"], next(n for n in grp if n.op == "conv1d_decode")
        K = int(gemms[0].params["K"])
        spec = f"gemv_fused K={K} pro=2 G=4 " + " ".join(
            f"N{i}={int(m.params['N'])} epi{i}={3 if i == 0 else (1 if m.params.get('cast') else 0)}" for i, m in enumerate(gemms)) + bpart
        # x, norm_w, then W, conv_state_in, conv_w, conv out, conv_state_new for the qkv rows and W, out for the others
        args = [norm.inputs[0].tensorName, norm.inputs[1].tensorName, gemms[0].inputs[1].tensorName, cv.inputs[1].tensorName,
                cv.inputs[2].tensorName, cv.outputs[0].tensorName, cv.outputs[1].tensorName]
        for m in gemms[1:]:
            args += [m.inputs[1].tensorName, m.outputs[0].tensorName]
        return KernelPlan(spec, name, args, [1, 1, 1], grp)
    if ops[0] == "rmsnorm" and ops[-1] == "swiglu":
        norm, gate, up, sw = grp
        N, K = int(gate.params["N"]), int(gate.params["K"])
        spec = f"gemv_fused K={K} pro=2 G=2 swiglu=1 N0={N} N1={N}" + bpart
        args = [norm.inputs[0].tensorName, norm.inputs[1].tensorName, gate.inputs[1].tensorName, up.inputs[1].tensorName,
                sw.outputs[0].tensorName]
        if batch >= Q8OUT_MIN_BATCH and N % 32 == 0:
            # the batched path writes the activation a second time as Q8_1, and the down projection reads that
            aux = sw.outputs[0].tensorName + ".q8_1"
            q8_of[sw.outputs[0].tensorName] = aux
            return KernelPlan(spec + " q8out=1", name, args + [aux], [1, 1, 1], grp, {aux: batch * (N // 32) * 36})
        return KernelPlan(spec, name, args, [1, 1, 1], grp)
    if ops[0] == "rmsnorm" and all(o == "gemm" for o in ops[1:]) and len(ops) > 1:
        norm, gemms = grp[0], grp[1:]
        K = int(gemms[0].params["K"])
        spec = f"gemv_fused K={K} pro=2 G={len(gemms)} " + " ".join(
            f"N{i}={int(m.params['N'])} epi{i}={1 if m.params.get('cast') else 0}" for i, m in enumerate(gemms)) + bpart
        args = [norm.inputs[0].tensorName, norm.inputs[1].tensorName]
        for m in gemms:
            args += [m.inputs[1].tensorName, m.outputs[0].tensorName]
        return KernelPlan(spec, name, args, [1, 1, 1], grp)
    if ops == ("gemm", "cast", "add"):
        m, c, a = grp
        cast_out = c.outputs[0].tensorName
        res = next(i.tensorName for i in a.inputs if i.tensorName != cast_out)
        N, K = int(m.params["N"]), int(m.params["K"])
        src = m.inputs[0].tensorName
        if src in raw_of:     # the activation is the raw block of a gdn_slabs op: its gated norm is this kernel's prologue
            aux, norm_w = raw_of[src]
            return KernelPlan(f"gemv_fused K={K} pro=3 G=1 N0={N} epi0=2" + bpart, name,
                              [aux, norm_w, m.inputs[1].tensorName, res, a.outputs[0].tensorName], [1, 1, 1], grp)
        if src in q8_of:      # the activation already exists as Q8_1 (written by a stand-alone rmsnorm_q8_1)
            spec, first = f"gemv_fused K={K} pro=0 G=1 N0={N} epi0=2" + bpart, q8_of[src]
        else:
            spec, first = f"gemv_fused K={K} pro=1 G=1 N0={N} epi0=2" + bpart, src
        return KernelPlan(spec, name, [first, m.inputs[1].tensorName, res, a.outputs[0].tensorName], [1, 1, 1], grp)
    if ops == ("conv1d_decode", "gdn_delta_rule"):
        cv, gd = grp
        spec = f"gdn_conv LVH={int(gd.params['LVH'])} LKD={int(gd.params['LKD'])} LVD={int(gd.params['LVD'])}" + bpart
        args = [cv.inputs[0].tensorName, cv.inputs[1].tensorName, cv.inputs[2].tensorName] + \
               [i.tensorName for i in gd.inputs[1:]] + [gd.outputs[0].tensorName, cv.outputs[1].tensorName, gd.outputs[1].tensorName]
        if batch < Q8OUT_MIN_BATCH:
            return KernelPlan(spec, name, args, [1, 1, 1], grp)
        # batched step: the threads that write the bf16 output also leave it as Q8_1 for out_proj (at batch 1 the
        # projection's own prologue does it as fast, and the recurrence kernel stays shorter)
        out, ZD = gd.outputs[0].tensorName, int(gd.params["ZD"])
        aux = out + ".q8_1"
        q8_of[out] = aux
        return KernelPlan(spec + " q8out=1", name, args + [aux], [1, 1, 1], grp, {aux: batch * (ZD // 32) * 36})
    if ops == ("qnorm", "rope", "knorm", "ropek", "fa2_attn"):
        qn, rp, kn, rk, fa = grp
        P = fa.params
        spec = (f"fa2_fused HD={int(P['HD'])} NH={int(P['NH'])} NKV={int(P['NKV'])} MAX_LEN={int(P['MAX_LEN'])} "
                f"ROT_HALF={int(rp.params['ROT_HALF'])}") + bpart + (" pos_dev=1" if device_scalars else "") + \
            ("" if attn_exact else " exact=0")
        args = [qn.inputs[0].tensorName, kn.inputs[0].tensorName, fa.inputs[2].tensorName, qn.inputs[1].tensorName,
                kn.inputs[1].tensorName, rp.inputs[1].tensorName, rp.inputs[2].tensorName, rp.inputs[3].tensorName,
                fa.inputs[4].tensorName, fa.inputs[5].tensorName, fa.outputs[0].tensorName]
        if batch < Q8OUT_MIN_BATCH:
            return KernelPlan(spec, name, args, [1, 1, 1], grp)
        out, n_out = fa.outputs[0].tensorName, int(P["NH"]) * int(P["HD"])
        aux = out + ".q8_1"
        q8_of[out] = aux
        return KernelPlan(spec + " q8out=1", name, args + [aux], [1, 1, 1], grp, {aux: batch * (n_out // 32) * 36})
    raise NotImplementedError(f"no fused kernel for the group {ops}")


def compilePartition(graph: Graph, ordered: Partition, batch: int = 1, device_scalars: bool = False, attn_exact: bool = True) -> list:
    """One KernelPlan per group.  Single nodes keep the reference's op and slot order; in a partition that has
    fused groups, a stand-alone rmsnorm whose readers are all matmuls also leaves its result as Q8_1 in an
    auxiliary buffer, and those matmuls read that instead of quantizing again."""
    fused = any(len(grp) > 1 for grp in ordered)
    q8_of: dict[str, str] = {}
    raw_of: dict[str, tuple] = {}       # output of a gdn_delta_rule node in slab form -> (its raw block, its norm weight)
    in_conv_group = {n.outputs[0].tensorName for grp in ordered if len(grp) == 6 for n in grp if n.op == "conv1d_decode"}
    plans = []
    for grp in ordered:
        if len(grp) != 1:
            plans.append(_group_plan(graph, grp, batch, device_scalars, q8_of, attn_exact, raw_of))
            continue
        n = grp[0]
        args = [i.tensorName for i in n.inputs] + [o.tensorName for o in n.outputs]
        bpart = f" batch={batch}" if batch != 1 else ""
        if fused and n.op == "gdn_delta_rule" and n.inputs[0].tensorName in in_conv_group:
            # slab form (fusedPartition put the convolution into the projections' group): the op leaves raw outputs, and
            # the one matmul that reads its output runs the gated norm in its prologue
            out = n.outputs[0].tensorName
            cons = graph.tensors[out].consumers
            if len(cons) == 1 and cons[0].op == "gemm" and cons[0].inputs[0].tensorName == out and int(cons[0].params["K"]) == 2048:
                aux = out + ".raw"
                raw_of[out] = (aux, n.inputs[6].tensorName)
                LVH = int(n.params["LVH"])
                spec = f"gdn_slabs LVH={LVH} LKD={int(n.params['LKD'])} LVD={int(n.params['LVD'])}" + bpart
                a = [i.tensorName for i in n.inputs]
                plans.append(KernelPlan(spec, f"gdn_slabs_{n.id}", a[:6] + [a[7], aux, n.outputs[1].tensorName], n.grid, grp,
                                        {aux: batch * (LVH * 128 * 8 + LVH * 32)}))
                continue
        if fused and n.op == "rmsnorm":
            out = n.outputs[0].tensorName
            cons = graph.tensors[out].consumers
            if cons and all(c.op == "gemm" and c.inputs[0].tensorName == out for c in cons):
                aux = out + ".q8_1"
                q8_of[out] = aux
                N = int(n.params["N"])
                plans.append(KernelPlan(f"rmsnorm_q8_1 N={N}" + bpart, f"rmsnorm_q8_1_{n.id}", args + [aux], n.grid, grp,
                                        {aux: batch * (N // 32) * 36}))
                continue
        if fused and n.op == "gemm" and n.inputs[0].tensorName in q8_of:
            N, K = int(n.params["N"]), int(n.params["K"])
            spec = f"gemv_fused K={K} pro=0 G=1 N0={N} epi0={1 if n.params.get('cast') else 0}" + bpart
            plans.append(KernelPlan(spec, f"gemv_{n.id}", [q8_of[n.inputs[0].tensorName], args[1], args[2]], n.grid, grp))
            continue
        plans.append(KernelPlan(node_spec(n, batch, device_scalars, attn_exact), f"{n.op}_{n.id}", args, n.grid, grp))
    return plans


def compileStep(graph: Graph, partition: Partition, batch: int = 1, device_scalars: bool = False, attn_exact: bool = True) -> CompiledStep:
    ordered = topoOrder(graph, partition)
    plans = compilePartition(graph, ordered, batch, device_scalars, attn_exact)
    cache: dict[str, rt.LoadedKernel] = {}
    schedule = []
    for p in plans:
        # handles own workspaces, so kernels with a workspace are not shared between nodes
        shareable = len(p.group) == 1 and p.group[0].op not in ("gemm", "fa2_attn", "argmax") and not p.spec.startswith("gemv_fused")
        if shareable and p.spec in cache:
            k = cache[p.spec]
        else:
            k = rt.compileAndLoad(p.spec, p.name, 4, p.name)
            if shareable:
                cache[p.spec] = k
        schedule.append((p, k))
    return CompiledStep(graph, schedule, batch, device_scalars)


# ---------------------------------------------------------------- token loop (src/runner.ts:116-162)
def runGraphDecode(compiled: CompiledStep, resolve: Callable[[str], int], initialToken: int, steps: int,
                   onToken: Callable | None = None, startPos: int = 0):
    """Greedy decode, one host launch per kernel per token; token id and position are scalars."""
    graph, schedule = compiled.graph, compiled.schedule
    argmax = next((n for n in graph.nodes if n.op == "argmax"), None)
    if argmax is None:
        raise RuntimeError("runGraphDecode: graph has no argmax node")
    idx_name, val_name = argmax.outputs[1].tensorName, argmax.outputs[0].tensorName
    tokens, logits = [], []
    for step in range(steps):
        token = initialToken if step == 0 else tokens[-1]
        pos = startPos + step
        for plan, k in schedule:
            args = [token if a == "token_id" else pos if a == "pos" else resolve(a) for a in plan.args]
            rc = rt.cuLaunch(k, plan.grid, [128, 1, 1], args)
            if rc != 0:
                raise rt.BunkerError(f"{plan.name}: {rt.last_error()} (rc={rc})")
        rt.cuSync()
        ibuf = np.zeros(1, np.int32); vbuf = np.zeros(1, np.float32)
        rt.cuDtoH(ibuf, resolve(idx_name), 4)
        rt.cuDtoH(vbuf, resolve(val_name), 4)
        tokens.append(int(ibuf[0])); logits.append(float(vbuf[0]))
        if onToken:
            onToken(int(ibuf[0]), float(vbuf[0]), step)
    return {"tokens": tokens, "logits": logits}


# ---------------------------------------------------------------- buffers (prototypes/decode_graph.ts:66-145)
_DT_BYTES = {"bf16": 2, "f32": 4, "i32": 4}


def tensor_bytes(t) -> int:
    n = 1
    for d in t.type.shape:
        n *= d
    if t.type.dtype == "q4_k":
        return n // 256 * 144
    return n * _DT_BYTES[t.type.dtype]


def state_key(name: str) -> str:
    """'n12_model.layers.0.conv_state_new' / 'model.layers.0.conv_state_in' -> 'model.layers.0.conv_state'."""
    if name.startswith("n") and "_" in name and name[1:name.index("_")].isdigit():
        name = name[name.index("_") + 1:]
    for suf in ("_in", "_new"):
        if name.endswith(suf):
            name = name[: -len(suf)]
    return name


class DecodeEnv:
    """Device buffers for one graph: weights, state (double-buffered), rope tables, intermediates.

    ``weights`` maps external weight names to numpy arrays (Q4_K bytes as uint8, bf16 as uint16
    bit patterns, f32); ``state`` maps state keys (``model.layers.L.conv_state`` ...) to initial
    numpy arrays.  K/V caches are single in-place buffers; conv and S state rotate between two
    buffers after every token unless ``inplace_state`` (both names then resolve to one buffer,
    which the kernels allow: every thread rewrites only what it read).
    """

    def __init__(self, graph: Graph, weights: dict, state: dict, inplace_state: bool = False,
                 device_weights: dict | None = None):
        self.graph = graph
        self.inplace = inplace_state
        self.ptr: dict[str, int] = {}
        self.aux: dict[str, int] = {}
        self.state_bufs: dict[str, list] = {}
        self.state_cur: dict[str, int] = {}
        self.non_rotating: set = set()
        self._owned: list = []
        for name, t in graph.tensors.items():
            if t.role == "scalar":
                continue
            if t.role == "weight":
                if device_weights is not None and name in device_weights:
                    self.ptr[name] = device_weights[name]       # already resident; owned by the caller
                    continue
                if name not in weights:
                    raise KeyError(f"DecodeEnv: no weight for '{name}'")
                arr = np.ascontiguousarray(weights[name])
                if arr.nbytes != tensor_bytes(t):
                    raise ValueError(f"DecodeEnv: '{name}' has {arr.nbytes} bytes, graph says {tensor_bytes(t)}")
                self.ptr[name] = self._own(rt.to_device(arr))
            elif t.role == "state":
                key = state_key(name)
                if key in self.state_bufs:
                    continue
                arr = np.ascontiguousarray(state[key])
                if arr.nbytes != tensor_bytes(t):
                    raise ValueError(f"DecodeEnv: state '{key}' has {arr.nbytes} bytes, graph says {tensor_bytes(t)}")
                a = self._own(rt.to_device(arr))
                if ".kv_k" in key or ".kv_v" in key or inplace_state:
                    self.state_bufs[key] = [a, a]
                    self.non_rotating.add(key)
                else:
                    b = self._own(rt.cuAlloc(arr.nbytes))
                    rt.cuMemset(b, 0, arr.nbytes)
                    self.state_bufs[key] = [a, b]
                self.state_cur[key] = 0
            else:
                self.ptr[name] = self._own(rt.cuAlloc(tensor_bytes(t)))
        rt.cuSync()

    def _own(self, p):
        self._owned.append(p)
        return p

    def weight_ptrs(self) -> dict:
        """Device pointers of the weights, to share them with another DecodeEnv (device_weights=...)."""
        return {n: p for n, p in self.ptr.items() if self.graph.tensors[n].role == "weight"}

    def add_aux(self, name: str, nbytes: int) -> int:
        """A buffer that only fused kernels of one compiled step see (not a tensor of the graph)."""
        if name not in self.aux:
            self.aux[name] = self._own(rt.cuAlloc(nbytes))
        return self.aux[name]

    def bind(self, compiled: "CompiledStep") -> None:
        for plan, _ in compiled.schedule:
            for name, nbytes in plan.aux.items():
                self.add_aux(name, nbytes)

    def resolve(self, name: str) -> int:
        if name in self.aux:
            return self.aux[name]
        t = self.graph.t(name)
        if t.role == "scalar":
            raise KeyError(f"resolve: scalar '{name}' is passed by the runner")
        if t.role == "state":
            key = state_key(name)
            cur = self.state_cur[key]
            is_new = name.endswith("_new")
            return self.state_bufs[key][1 - cur if is_new else cur]
        return self.ptr[name]

    def rotateState(self):
        for key in self.state_bufs:
            if key not in self.non_rotating:
                self.state_cur[key] = 1 - self.state_cur[key]

    def read_state(self, key: str, shape, dtype) -> np.ndarray:
        return rt.from_device(self.state_bufs[key][self.state_cur[key]], shape, dtype)

    def close(self):
        for p in self._owned:
            rt.cuFree(p)
        self._owned = []


# ---------------------------------------------------------------- device-resident loop
def cache_capacity(graph: Graph):
    """Tokens a sequence's KV cache (and the rope tables) hold: MAX_LEN of the graph's attention nodes, None without any."""
    caps = [int(n.params["MAX_LEN"]) for n in graph.nodes if "MAX_LEN" in n.params]
    return min(caps) if caps else None


class DeviceLoop:
    """Greedy decode with token ids and positions in device memory and the step in a HIP graph.

    One replay = one token for every sequence of the batch: the step's kernels, then a small
    kernel that feeds argmax's indices back as the next token ids, advances the positions and
    appends the tokens to a device-side history.  State is updated in place.
    """

    def __init__(self, graph: Graph, env: DecodeEnv, batch: int, start_tokens, start_pos, max_steps: int,
                 partition: Partition | None = None, use_graph: bool = True, feed: bool = True, attn_exact: bool = True):
        if not env.inplace:
            raise ValueError("DeviceLoop needs DecodeEnv(inplace_state=True)")
        ids = np.asarray(start_tokens, np.int32).reshape(batch)
        pos = np.broadcast_to(np.asarray(start_pos, np.int32), (batch,)).copy()
        # Positions advance on the device, where no launcher can check them: the whole run must fit the cache before
        # anything is launched.  (The kernels skip a cache write past the capacity, but the tokens would be wrong.)
        max_len = cache_capacity(graph)
        if max_steps < 1:
            raise ValueError(f"DeviceLoop: max_steps={max_steps} must be at least 1")
        if int(pos.min()) < 0:
            raise ValueError(f"DeviceLoop: negative start position {int(pos.min())}")
        if max_len is not None and int(pos.max()) + max_steps > max_len:
            raise ValueError(f"DeviceLoop: start position {int(pos.max())} + {max_steps} steps exceeds the KV capacity "
                             f"MAX_LEN={max_len}")
        self.graph, self.env, self.batch, self.max_steps = graph, env, batch, max_steps
        self.compiled = compileStep(graph, partition or choosePartition(graph), batch, device_scalars=True, attn_exact=attn_exact)
        env.bind(self.compiled)
        self.d_ids = rt.to_device(ids)
        self.d_pos = rt.to_device(pos)
        self.d_hist = rt.cuAlloc(max_steps * batch * 8)
        self.d_count = rt.to_device(np.zeros(batch, np.int32))
        argmax = next(n for n in graph.nodes if n.op == "argmax")
        self.idx_ptr = env.resolve(argmax.outputs[1].tensorName)
        self.val_ptr = env.resolve(argmax.outputs[0].tensorName)
        max_pos = max_len if max_len is not None else 2**31 - 1
        self.launches = []
        for plan, k in self.compiled.schedule:
            args = [self.d_ids if a == "token_id" else self.d_pos if a == "pos" else env.resolve(a) for a in plan.args]
            self.launches.append((k, plan, args))
        # Between two tokens: argmax's second stage, the token feedback and the next token's embedding are one launch
        # (argmax_feed) when the step begins with the embed node and ends with the argmax node on their own; the embed
        # launch then runs once, in front of the first step.  Otherwise argmax, then `advance`.
        self.first_only = []
        first, last = self.launches[0][1], self.launches[-1][1]
        if feed and len(first.group) == 1 and first.group[0].op == "embed" and len(last.group) == 1 and last.group[0].op == "argmax":
            emb = first.group[0]
            H, V = int(emb.params["H"]), int(emb.params["VOCAB"])
            k_feed = rt.compileAndLoad(f"argmax_feed VOCAB={V} H={H} batch={batch} max_steps={max_steps} max_pos={max_pos}")
            self.first_only = [self.launches[0]]
            rt.unloadKernel(self.launches[-1][0])
            self.launches = self.launches[1:-1]
            self.launches.append((k_feed, None, [env.resolve(argmax.inputs[0].tensorName), self.val_ptr, self.idx_ptr, self.d_ids, self.d_pos,
                                                 self.d_hist, self.d_count, env.resolve(emb.inputs[0].tensorName),
                                                 env.resolve(emb.outputs[0].tensorName)]))
        else:
            self.k_adv = rt.compileAndLoad(f"advance batch={batch} max_steps={max_steps} max_pos={max_pos}")
            self.launches.append((self.k_adv, None, [self.idx_ptr, self.val_ptr, self.d_ids, self.d_pos, self.d_hist, self.d_count]))
        self.graph_exec = None
        self.use_graph = use_graph
        self.steps_done = 0

    def _enqueue(self, first: bool = False):
        for k, plan, args in (self.first_only if first else []) + self.launches:
            rc = rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], args)
            if rc != 0:
                raise rt.BunkerError(f"{plan.name if plan else 'advance'}: {rt.last_error()} (rc={rc})")

    def step(self, n: int = 1):
        for _ in range(n):
            if self.steps_done >= self.max_steps:
                raise RuntimeError("DeviceLoop: history is full")
            if not self.launches:
                raise RuntimeError("DeviceLoop: closed")
            if self.graph_exec is not None:
                self.graph_exec.launch()
            else:
                # the first token runs eagerly (it also loads every kernel); the recording happens after it
                self._enqueue(first=self.steps_done == 0)
                if self.use_graph:
                    rt.cuSync()
                    with rt.Graph() as gr:
                        self._enqueue()
                    self.graph_exec = gr
            self.steps_done += 1

    def close(self):
        """Release what the loop owns on the device: the recorded graph, the kernel handles with their workspaces and
        the four small buffers.  The DecodeEnv (weights, state) is the caller's."""
        rt.cuSync()
        if self.graph_exec is not None:
            self.graph_exec.destroy()
            self.graph_exec = None
        seen = set()
        for k, _, _ in self.first_only + self.launches:
            if k.fn not in seen:
                seen.add(k.fn)
                rt.unloadKernel(k)
        self.launches = []
        self.first_only = []
        for p in (self.d_ids, self.d_pos, self.d_hist, self.d_count):
            if p:
                rt.cuFree(p)
        self.d_ids = self.d_pos = self.d_hist = self.d_count = 0

    def tokens(self):
        """(tokens int32 [steps, batch], logits f32 [steps, batch]) generated so far."""
        rt.cuSync()
        raw = rt.from_device(self.d_hist, (self.max_steps, self.batch, 2), np.int32)[: self.steps_done]
        return raw[..., 0].copy(), raw[..., 1].copy().view(np.float32)
