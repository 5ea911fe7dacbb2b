// specs.ts — the graph-level half of the drop-in: what src/fusion.ts:480-498 (compilePartition / loadPartition) and
// prototypes/decode_graph.ts:66-145 (state buffers, rope tables, resolve) do in the reference, for libbunker_hip.so.
//
// Drop next to hip.ts.  src/model.ts (buildModelGraph) and src/runner.ts (topoOrder, runGraphDecode) stay as they
// are; where the reference turns a group of graph nodes into TTIR text (codegenGroup) this file turns it into an op
// spec string for compileAndLoad of hip.ts — the op name of src/model.ts plus the constants the emitters baked into the
// kernel text — and into the slot list cuLaunch packs (node inputs in declared order, then outputs,
// src/fusion.ts:371-401).  Two partitions are served: every node its own kernel (src/runner.ts:40-49), and the fused
// groups below, which are the ones that pay on MI355X.
//
// The literal tables SPEC_KEYS, FUSED_SPECS and SPEC_SUFFIX are the contract with the library: tests/test_ts_specs.py
// expands them (plain ${name} substitution) for all 424 nodes and all fused groups of the synthetic model and compares
// with tests/golden/node_specs.json, which is written from the Python host layer that runs against the GPU.
import { compileAndLoad, cuAlloc, cuHtoD, type LoadedKernel } from "./hip";

// ---- the reference's graph types (src/fusion.ts:47-117), as far as this file reads them
export interface NodeIO { name: string; tensorName: string; role: string; }
export interface GraphNode { id: number; op: string; inputs: NodeIO[]; outputs: NodeIO[]; grid: number[]; params: Record<string, number | boolean | string>; }
export interface Tensor { name: string; role: string; producer: GraphNode | null; consumers: GraphNode[]; }
export interface Graph { nodes: GraphNode[]; tensors: Map<string, Tensor>; }
export interface KernelPlan { spec: string; name: string; args: string[]; grid: number[]; group: GraphNode[]; aux: Record<string, number>; }
export interface Dims { H: number; VOCAB: number; NL: number; FAI: number; INTER: number; NH: number; NKV: number; HD: number;
                        LKH: number; LVH: number; LKD: number; LVD: number; MAX_LEN: number; ROT_DIM: number; }

// ---- constants of an op that go into its spec, in this order (the library reads them by name)
export const SPEC_KEYS: Record<string, string[]> = {
  "embed": ["H", "VOCAB"],
  "rmsnorm": ["N"],
  "gemm": ["N", "K"],
  "cast": ["N"],
  "add": ["N"],
  "swiglu": ["N"],
  "conv1d_decode": ["QKVD"],
  "gdn_delta_rule": ["LVH", "LKD", "LVD"],
  "qnorm": ["HD", "NH"],
  "knorm": ["HD", "NKV"],
  "rope": ["HD", "NH", "ROT_HALF", "MAX_LEN"],
  "ropek": ["HD", "NKV", "ROT_HALF", "MAX_LEN"],
  "fa2_attn": ["HD", "NH", "NKV", "MAX_LEN"],
  "argmax": ["VOCAB"],
};

// ---- specs of the fused groups, keyed by the ops of the group joined with "+" ("gemm*" = one to four matmuls)
export const FUSED_SPECS: Record<string, string> = {
  "rmsnorm+gemm+gemm+swiglu": "gemv_fused K=${K} pro=2 G=2 swiglu=1 N0=${N} N1=${N}",
  "rmsnorm+gemm*": "gemv_fused K=${K} pro=2 G=${G}${MATS}",
  "mat": " N${i}=${N} epi${i}=${EPI}",
  "gemm+cast+add": "gemv_fused K=${K} pro=${PRO} G=1 N0=${N} epi0=2",
  "conv1d_decode+gdn_delta_rule": "gdn_conv LVH=${LVH} LKD=${LKD} LVD=${LVD}",
  // slab form of a GDN layer (batch <= SLAB_MAX_BATCH): conv1d is the last step of the qkv rows (epi0=3), the
  // recurrence runs in four column slabs per head and leaves raw outputs, the out_proj group runs its gated norm (pro=3)
  "rmsnorm+gemm*+conv1d_decode": "gemv_fused K=${K} pro=2 G=4${MATS}",
  "gdn_slabs": "gdn_slabs LVH=${LVH} LKD=${LKD} LVD=${LVD}",
  "gemm+cast+add@raw": "gemv_fused K=${K} pro=3 G=1 N0=${N} epi0=2",
  "qnorm+rope+knorm+ropek+fa2_attn": "fa2_fused HD=${HD} NH=${NH} NKV=${NKV} MAX_LEN=${MAX_LEN} ROT_HALF=${ROT_HALF}",
  "rmsnorm_q8_1": "rmsnorm_q8_1 N=${N}",
  "gemm@q8_1": "gemv_fused K=${K} pro=0 G=1 N0=${N} epi0=${EPI}",
};

// ---- optional tails of a spec, appended in this order
export const SPEC_SUFFIX: Record<string, string> = {
  "cast": " cast=1",            // gemm nodes with params.cast
  "batch": " batch=${batch}",   // batch != 1
  "ids_dev": " ids_dev=1",      // embed, token ids in device memory
  "pos_dev": " pos_dev=1",      // rope, ropek, fa2_attn, fa2_fused: positions in device memory
  "exact0": " exact=0",         // fa2_attn, fa2_fused: the bf16 matrix-instruction attention instead of the f64 form
  "q8out": " q8out=1",          // batch >= Q8OUT_MIN_BATCH: the producer also leaves its output as Q8_1 blocks
};

export const Q8OUT_MIN_BATCH = 8;      // from this batch on producers also emit Q8_1 and the matmuls behind them read it
export const SLAB_MAX_BATCH = 7;       // up to this batch a GDN layer with ZD = 2048 and projection rows of 1024 / 2048 takes the slab form
export const LM_HEAD_ROWS = 32768;     // matmuls with more rows keep the stand-alone norm + quantizer

function fill(template: string, vars: Record<string, number | string>): string {
  return template.replace(/\$\{(\w+)\}/g, (_, k) => String(vars[k]));
}
const int = (v: number | boolean | string) => Math.trunc(Number(v));

/** Spec of a single node: op, its constants, then the tails that apply (runner.node_spec of the Python host). */
export function nodeSpec(n: GraphNode, batch = 1, deviceScalars = false, attnExact = true): string {
  let s = [n.op, ...SPEC_KEYS[n.op].map((k) => `${k}=${int(n.params[k])}`)].join(" ");
  if (n.op === "gemm" && n.params.cast) s += SPEC_SUFFIX.cast;
  if (batch !== 1) s += fill(SPEC_SUFFIX.batch, { batch });
  if (deviceScalars && n.op === "embed") s += SPEC_SUFFIX.ids_dev;
  if (deviceScalars && (n.op === "rope" || n.op === "ropek" || n.op === "fa2_attn")) s += SPEC_SUFFIX.pos_dev;
  if (n.op === "fa2_attn" && !attnExact) s += SPEC_SUFFIX.exact0;
  return s;
}

const tn = (io: NodeIO) => io.tensorName;

/** Spec and slot list of a fused group (the counterpart of codegenGroup for the groups fusedPartition forms). */
export function groupPlan(grp: GraphNode[], batch: number, deviceScalars: boolean, q8Of: Map<string, string>, attnExact = true,
                          rawOf: Map<string, [string, string]> = new Map()): KernelPlan {
  const ops = grp.map((n) => n.op);
  const key = ops.join("+");
  const bpart = batch !== 1 ? fill(SPEC_SUFFIX.batch, { batch }) : "";
  const name = `${key}_${grp[0].id}`;
  const plan = (spec: string, args: string[], aux: Record<string, number> = {}): KernelPlan => ({ spec, name, args, grid: [1, 1, 1], group: grp, aux });
  if (key === "rmsnorm+gemm+gemm+swiglu") {
    const [norm, gate, up, sw] = grp;
    const N = int(gate.params.N), K = int(gate.params.K);
    const spec = fill(FUSED_SPECS[key], { K, N }) + bpart;
    const args = [tn(norm.inputs[0]), tn(norm.inputs[1]), tn(gate.inputs[1]), tn(up.inputs[1]), tn(sw.outputs[0])];
    if (batch >= Q8OUT_MIN_BATCH && N % 32 === 0) {
      const aux = tn(sw.outputs[0]) + ".q8_1";
      q8Of.set(tn(sw.outputs[0]), aux);
      return plan(spec + SPEC_SUFFIX.q8out, [...args, aux], { [aux]: batch * (N / 32) * 36 });
    }
    return plan(spec, args);
  }
  if (ops[0] === "rmsnorm" && ops.length === 6 && ops.filter((o) => o === "gemm").length === 4 && ops.includes("conv1d_decode")) {
    // norm + qkv, z, a, b + conv1d_decode over the qkv rows (the group is ordered by node id: the conv node sits between the matmuls)
    const norm = grp[0], gemms = grp.filter((n) => n.op === "gemm"), cv = grp.find((n) => n.op === "conv1d_decode")!;
    const MATS = gemms.map((m, i) => fill(FUSED_SPECS.mat, { i, N: int(m.params.N), EPI: i === 0 ? 3 : (m.params.cast ? 1 : 0) })).join("");
    // x, norm_w, then W, conv_state_in, conv_w, conv out, conv_state_new for the qkv rows and W, out for the others
    const args = [tn(norm.inputs[0]), tn(norm.inputs[1]), tn(gemms[0].inputs[1]), tn(cv.inputs[1]), tn(cv.inputs[2]), tn(cv.outputs[0]), tn(cv.outputs[1])];
    for (const m of gemms.slice(1)) args.push(tn(m.inputs[1]), tn(m.outputs[0]));
    return plan(fill(FUSED_SPECS["rmsnorm+gemm*+conv1d_decode"], { K: int(gemms[0].params.K), MATS }) + bpart, args);
  }
  if (ops[0] === "rmsnorm" && ops.length > 1 && ops.slice(1).every((o) => o === "gemm")) {
    const [norm, ...gemms] = grp;
    const K = int(gemms[0].params.K);
    const MATS = gemms.map((m, i) => fill(FUSED_SPECS.mat, { i, N: int(m.params.N), EPI: m.params.cast ? 1 : 0 })).join("");
    const args = [tn(norm.inputs[0]), tn(norm.inputs[1])];
    for (const m of gemms) args.push(tn(m.inputs[1]), tn(m.outputs[0]));
    return plan(fill(FUSED_SPECS["rmsnorm+gemm*"], { K, G: gemms.length, MATS }) + bpart, args);
  }
  if (key === "gemm+cast+add") {
    const [m, c, a] = grp;
    const castOut = tn(c.outputs[0]);
    const res = tn(a.inputs.find((i) => i.tensorName !== castOut)!);
    const N = int(m.params.N), K = int(m.params.K), src = tn(m.inputs[0]);
    if (rawOf.has(src)) {
      // the activation is the raw block of a gdn_slabs op: its gated norm is this kernel's prologue
      const [aux, normW] = rawOf.get(src)!;
      return plan(fill(FUSED_SPECS["gemm+cast+add@raw"], { K, N }) + bpart, [aux, normW, tn(m.inputs[1]), res, tn(a.outputs[0])]);
    }
    // the activation already exists as Q8_1 (written by a stand-alone rmsnorm_q8_1 or a q8out producer): pro=0
    const first = q8Of.get(src) ?? src;
    const spec = fill(FUSED_SPECS[key], { K, N, PRO: q8Of.has(src) ? 0 : 1 }) + bpart;
    return plan(spec, [first, tn(m.inputs[1]), res, tn(a.outputs[0])]);
  }
  if (key === "conv1d_decode+gdn_delta_rule") {
    const [cv, gd] = grp;
    const spec = fill(FUSED_SPECS[key], { LVH: int(gd.params.LVH), LKD: int(gd.params.LKD), LVD: int(gd.params.LVD) }) + bpart;
    const args = [tn(cv.inputs[0]), tn(cv.inputs[1]), tn(cv.inputs[2]), ...gd.inputs.slice(1).map(tn), tn(gd.outputs[0]),
                  tn(cv.outputs[1]), tn(gd.outputs[1])];
    if (batch < Q8OUT_MIN_BATCH) return plan(spec, args);
    const out = tn(gd.outputs[0]), aux = out + ".q8_1";
    q8Of.set(out, aux);
    return plan(spec + SPEC_SUFFIX.q8out, [...args, aux], { [aux]: batch * (int(gd.params.ZD) / 32) * 36 });
  }
  if (key === "qnorm+rope+knorm+ropek+fa2_attn") {
    const [qn, rp, kn, , fa] = grp;
    const P = fa.params;
    const spec = fill(FUSED_SPECS[key], { HD: int(P.HD), NH: int(P.NH), NKV: int(P.NKV), MAX_LEN: int(P.MAX_LEN), ROT_HALF: int(rp.params.ROT_HALF) }) +
      bpart + (deviceScalars ? SPEC_SUFFIX.pos_dev : "") + (attnExact ? "" : SPEC_SUFFIX.exact0);
    // q|gate, k, v, q_norm.weight, k_norm.weight, rope_cos, rope_sin, pos, kv_k, kv_v, out
    const args = [tn(qn.inputs[0]), tn(kn.inputs[0]), tn(fa.inputs[2]), tn(qn.inputs[1]), tn(kn.inputs[1]), tn(rp.inputs[1]),
                  tn(rp.inputs[2]), tn(rp.inputs[3]), tn(fa.inputs[4]), tn(fa.inputs[5]), tn(fa.outputs[0])];
    if (batch < Q8OUT_MIN_BATCH) return plan(spec, args);
    const out = tn(fa.outputs[0]), aux = out + ".q8_1";
    q8Of.set(out, aux);
    return plan(spec + SPEC_SUFFIX.q8out, [...args, aux], { [aux]: batch * ((int(P.NH) * int(P.HD)) / 32) * 36 });
  }
  throw new Error(`no fused kernel for the group ${key}`);
}

/** src/fusion.ts:480-491: one KernelPlan per group of an ordered partition. */
export function compilePartition(graph: Graph, ordered: GraphNode[][], batch = 1, deviceScalars = false, attnExact = true): KernelPlan[] {
  const fused = ordered.some((g) => g.length > 1);
  const q8Of = new Map<string, string>();
  const rawOf = new Map<string, [string, string]>();    // output of a gdn_delta_rule node in slab form -> [raw block, norm weight]
  const inConvGroup = new Set<string>();
  for (const g of ordered) if (g.length === 6) for (const n of g) if (n.op === "conv1d_decode") inConvGroup.add(tn(n.outputs[0]));
  const plans: KernelPlan[] = [];
  for (const grp of ordered) {
    if (grp.length !== 1) { plans.push(groupPlan(grp, batch, deviceScalars, q8Of, attnExact, rawOf)); continue; }
    const n = grp[0];
    const args = [...n.inputs.map(tn), ...n.outputs.map(tn)];
    const bpart = batch !== 1 ? fill(SPEC_SUFFIX.batch, { batch }) : "";
    if (fused && n.op === "gdn_delta_rule" && inConvGroup.has(tn(n.inputs[0]))) {
      // slab form: raw outputs; the one matmul that reads the op's output runs the gated norm in its prologue
      const out = tn(n.outputs[0]);
      const cons = graph.tensors.get(out)!.consumers;
      if (cons.length === 1 && cons[0].op === "gemm" && cons[0].inputs[0].tensorName === out && int(cons[0].params.K) === 2048) {
        const aux = out + ".raw", LVH = int(n.params.LVH), a = n.inputs.map(tn);
        rawOf.set(out, [aux, a[6]]);
        plans.push({ spec: fill(FUSED_SPECS.gdn_slabs, { LVH, LKD: int(n.params.LKD), LVD: int(n.params.LVD) }) + bpart, name: `gdn_slabs_${n.id}`,
                     args: [...a.slice(0, 6), a[7], aux, tn(n.outputs[1])], grid: n.grid, group: grp, aux: { [aux]: batch * (LVH * 128 * 8 + LVH * 32) } });
        continue;
      }
    }
    if (fused && n.op === "rmsnorm") {
      // a stand-alone norm whose readers are all matmuls also leaves its result as Q8_1; those matmuls read that
      const out = tn(n.outputs[0]);
      const cons = graph.tensors.get(out)!.consumers;
      if (cons.length && cons.every((c) => c.op === "gemm" && c.inputs[0].tensorName === out)) {
        const aux = out + ".q8_1", N = int(n.params.N);
        q8Of.set(out, aux);
        plans.push({ spec: fill(FUSED_SPECS.rmsnorm_q8_1, { N }) + bpart, name: `rmsnorm_q8_1_${n.id}`, args: [...args, aux], grid: n.grid,
                     group: grp, aux: { [aux]: batch * (N / 32) * 36 } });
        continue;
      }
    }
    if (fused && n.op === "gemm" && q8Of.has(n.inputs[0].tensorName)) {
      const spec = fill(FUSED_SPECS["gemm@q8_1"], { K: int(n.params.K), N: int(n.params.N), EPI: n.params.cast ? 1 : 0 }) + bpart;
      plans.push({ spec, name: `gemv_${n.id}`, args: [q8Of.get(n.inputs[0].tensorName)!, args[1], args[2]], grid: n.grid, group: grp, aux: {} });
      continue;
    }
    plans.push({ spec: nodeSpec(n, batch, deviceScalars, attnExact), name: `${n.op}_${n.id}`, args, grid: n.grid, group: grp, aux: {} });
  }
  return plans;
}

/** src/fusion.ts:493-498: a kernel handle per plan (nothing is compiled: the library looks the op up). */
export function loadPartition(plans: KernelPlan[]): { plan: KernelPlan; kernel: LoadedKernel }[] {
  return plans.map((plan) => ({ plan, kernel: compileAndLoad(plan.spec, plan.name, 4, plan.name) }));
}

// ---- buffers of prototypes/decode_graph.ts:66-145 that differ from the reference's: sizes in bytes per layer
export const PAGE_TOKENS = 16;
/** Recurrent and cache state of one layer for `batch` sequences.  K page (p, h): bf16 [16 tok][HD]; V page (p, h): bf16
 * [HD][16 tok] (dim-major), both at element offset (p * NKV + h) * 16 * HD; a sequence owns MAX_LEN / 16 pages. */
export function stateBytes(D: Dims, batch: number) {
  const QKVD = 2 * D.LKH * D.LKD + D.LVH * D.LVD;
  return {
    conv_state: batch * 3 * QKVD * 2,                    // bf16 [B, 3, QKVD]
    s_state: batch * D.LVH * D.LKD * D.LVD * 4,          // f32  [B, LVH, LKD, LVD]
    kv_k: batch * D.NKV * D.MAX_LEN * D.HD * 2,          // bf16 pages, see above
    kv_v: batch * D.NKV * D.MAX_LEN * D.HD * 2,
    rope_table: D.MAX_LEN * (D.ROT_DIM / 2) * 4,         // f32 [MAX_LEN, ROT_DIM / 2], cos and sin each
    block_table_entries: batch * (D.MAX_LEN / PAGE_TOKENS),
  };
}
/** cos / sin of prototypes/decode_graph.ts:120-131 (theta^(-2 i / ROT_DIM), f64 then f32), uploaded once. */
export function ropeTables(D: Dims, theta = 1e7): { cos: bigint; sin: bigint } {
  const half = D.ROT_DIM / 2, cos = new Float32Array(D.MAX_LEN * half), sin = new Float32Array(D.MAX_LEN * half);
  for (let p = 0; p < D.MAX_LEN; p++)
    for (let i = 0; i < half; i++) {
      const a = p * Math.pow(theta, (-2 * i) / D.ROT_DIM);
      cos[p * half + i] = Math.cos(a); sin[p * half + i] = Math.sin(a);
    }
  const dc = cuAlloc(cos.byteLength), ds = cuAlloc(sin.byteLength);
  cuHtoD(dc, cos.buffer); cuHtoD(ds, sin.buffer);
  return { cos: dc, sin: ds };
}
