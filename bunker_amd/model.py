"""Whole-model declaration of a Qwen3.5-style decode step as a graph.

Counterpart of src/model.ts: the same node sequence per layer — embed, then 24 x
(rmsnorm, [GDN: qkv, z, conv1d, a, b, gdn_delta_rule, out_proj | FA: q, k, v, qnorm, rope,
knorm, ropek, fa2_attn, o_proj], cast, add, rmsnorm, gate, up, swiglu, down, cast, add),
final rmsnorm, lm_head, argmax (src/model.ts:46-204) — the same tensor names for weights and
state, the same argument order per node.  Differences, all on purpose:

* dimensions are a parameter (``Dims``): ``SYNTH`` is the synthetic model of the benchmark
  (hidden 2048, FFN 6144, vocab 151936, 16 query / 2 KV heads), ``REFERENCE`` holds the
  constants of src/model.ts:14-18;
* linear weights are Q4_K (``dtype "q4_k"``, ``[N, K]`` row-major in 144-byte super-blocks) and
  every ``gemm`` node is served by "quantize A to Q8_1, Q4_K x Q8_1 GEMV";
* the KV cache is shared by the query heads of a group and paged: K ``[MAX_LEN/16 pages][NKV]
  [16][HD]``, V ``[pages][NKV][HD][16]`` (the reference keeps one unpaged copy per query head,
  src/emitters.ts:202);
* lm_head is its own Q4_K matrix instead of the tied embedding (prototypes/decode_graph.py:100);
* every activation and state tensor has a leading batch dimension.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace

from .graph import Graph, TensorType, row_major


@dataclass(frozen=True)
class Dims:
    H: int = 2048
    VOCAB: int = 151936
    NL: int = 24
    FAI: int = 4               # every FAI-th layer (layer % FAI == FAI-1) is full attention
    INTER: int = 6144
    NH: int = 16
    NKV: int = 2
    HD: int = 256
    LKH: int = 16              # GDN key heads
    LVH: int = 16              # GDN value heads
    LKD: int = 128
    LVD: int = 128
    MAX_LEN: int = 4352        # KV capacity in tokens (multiple of 16)
    ROT_DIM: int = 64
    EPS: float = 1e-6
    ROPE_THETA: float = 1e7

    @property
    def QKVD(self): return 2 * self.LKH * self.LKD + self.LVH * self.LVD
    @property
    def ZD(self): return self.LVH * self.LVD
    @property
    def QGATE(self): return 2 * self.NH * self.HD
    @property
    def KV_DIM(self): return self.NKV * self.HD
    @property
    def ROT_HALF(self): return self.ROT_DIM // 2

    def is_full_attention(self, layer: int) -> bool:
        return layer % self.FAI == self.FAI - 1

    def __post_init__(self):
        # a sequence owns MAX_LEN/16 whole pages of the cache; the kernels size block-table rows from it
        if self.MAX_LEN < 16 or self.MAX_LEN % 16 != 0:
            raise ValueError(f"Dims: MAX_LEN={self.MAX_LEN} must be a positive multiple of the 16-token page")


SYNTH = Dims()
# src/model.ts:14-18
REFERENCE = Dims(H=1024, VOCAB=248320, NL=24, FAI=4, INTER=3584, NH=8, NKV=2, HD=256, LKH=16, LVH=16,
                 LKD=128, LVD=128, MAX_LEN=128)
# a small model with the same structure, for tests that run the CPU checker end to end
TINY = Dims(H=256, VOCAB=1024, NL=4, FAI=4, INTER=512, NH=16, NKV=2, HD=256, LKH=2, LVH=2, MAX_LEN=64)


def L(layer: int) -> str:
    return f"model.layers.{layer}"


def buildModelGraph(D: Dims = SYNTH, batch: int = 1) -> Graph:
    """The decode graph for ONE token step of ``batch`` independent sequences."""
    g = Graph()
    B = batch

    def act(n, dtype="bf16"):
        return row_major([B, n], dtype)

    def weight(name, shape, dtype="bf16"):
        return g.input(name, row_major(shape, dtype), "weight")

    def gemm(a, wname, N, K, cast):
        n = g.node("gemm", [(a, "A"), (weight(wname, [N, K], "q4_k"), "B")],
                   [("out", act(N, "bf16" if cast else "f32"))], [1, math.ceil(N / 64), 1],
                   {"M": 1, "N": N, "K": K, **({"cast": True} if cast else {})})
        return g.out(n)

    def residual(x_f32, h, N, order):
        c = g.node("cast", [(x_f32, "x")], [("out", act(N))], [1, math.ceil(N / 64), 1], {"to": "bf16", "N": N})
        ins = [(g.out(c), "a"), (h, "b")] if order == "attn" else [(h, "a"), (g.out(c), "b")]
        a = g.node("add", ins, [("out", act(N))], [1, math.ceil(N / 64), 1], {"N": N})
        return g.out(a)

    scalar = TensorType([], "i32", [])
    Tk = g.input("token_id", scalar, "scalar")
    Pos = g.input("pos", scalar, "scalar")
    emb = g.node("embed", [(weight("embed.weight", [D.VOCAB, D.H]), "E"), (Tk, "id")], [("out", act(D.H))],
                 [1, 1, 1], {"H": D.H, "VOCAB": D.VOCAB})
    h = g.out(emb)

    for layer in range(D.NL):
        pre = L(layer)
        normed = g.out(g.node("rmsnorm", [(h, "x"), (weight(f"{pre}.input_layernorm.weight", [D.H]), "w")],
                              [("out", act(D.H))], [1, 1, 1], {"N": D.H}))
        if not D.is_full_attention(layer):
            la = f"{pre}.linear_attn"
            qkv = gemm(normed, f"{la}.in_proj_qkv.weight", D.QKVD, D.H, True)
            z = gemm(normed, f"{la}.in_proj_z.weight", D.ZD, D.H, True)
            conv_state = g.input(f"{pre}.conv_state_in", row_major([B, 3, D.QKVD], "bf16"), "state")
            conv = g.node("conv1d_decode",
                          [(qkv, "qkv"), (conv_state, "state"), (weight(f"{la}.conv1d.weight", [D.QKVD, 4]), "w")],
                          [("out", act(D.QKVD)), (f"{pre}.conv_state_new", row_major([B, 3, D.QKVD], "bf16"), "state")],
                          [math.ceil(D.QKVD / 1024), 1, 1], {"QKVD": D.QKVD})
            a_p = gemm(normed, f"{la}.in_proj_a.weight", D.LVH, D.H, False)
            b_p = gemm(normed, f"{la}.in_proj_b.weight", D.LVH, D.H, False)
            s_type = row_major([B, D.LVH, D.LKD, D.LVD], "f32")
            gdn = g.node("gdn_delta_rule",
                         [(g.out(conv), "conv_out"), (z, "z"), (weight(f"{la}.A_log", [D.LVH], "f32"), "A_log"),
                          (weight(f"{la}.dt_bias", [D.LVH]), "dt_bias"), (a_p, "a_p"), (b_p, "b_p"),
                          (weight(f"{la}.norm.weight", [D.LVD], "f32"), "norm_w"),
                          (g.input(f"{pre}.s_state_in", s_type, "state"), "s_state")],
                         [("out", act(D.ZD)), (f"{pre}.s_state_new", s_type, "state")], [D.LVH, 1, 1],
                         {"LVH": D.LVH, "LKD": D.LKD, "LVD": D.LVD, "QKVD": D.QKVD, "KEYDIM": D.LKH * D.LKD, "ZD": D.ZD})
            proj = gemm(g.out(gdn), f"{la}.out_proj.weight", D.H, D.ZD, False)
        else:
            sa = f"{pre}.self_attn"
            qp = gemm(normed, f"{sa}.q_proj.weight", D.QGATE, D.H, True)
            kp = gemm(normed, f"{sa}.k_proj.weight", D.KV_DIM, D.H, True)
            vp = gemm(normed, f"{sa}.v_proj.weight", D.KV_DIM, D.H, True)
            rope_cos = g.tensors.get("rope_cos") or weight("rope_cos", [D.MAX_LEN, D.ROT_HALF], "f32")
            rope_sin = g.tensors.get("rope_sin") or weight("rope_sin", [D.MAX_LEN, D.ROT_HALF], "f32")
            qn = g.node("qnorm", [(qp, "q"), (weight(f"{sa}.q_norm.weight", [D.HD]), "w")],
                        [("out", act(D.NH * D.HD))], [D.NH, 1, 1], {"HD": D.HD, "NH": D.NH})
            # rope / ropek rotate the norm outputs in place and declare no output (src/model.ts:133-143)
            g.node("rope", [(g.out(qn), "Q"), (rope_cos, "C"), (rope_sin, "S"), (Pos, "P")], [], [D.NH, 1, 1],
                   {"HD": D.HD, "NH": D.NH, "ROT_HALF": D.ROT_HALF, "MAX_LEN": D.MAX_LEN})
            kn = g.node("knorm", [(kp, "k"), (weight(f"{sa}.k_norm.weight", [D.HD]), "w")],
                        [("out", act(D.KV_DIM))], [D.NKV, 1, 1], {"HD": D.HD, "NKV": D.NKV})
            g.node("ropek", [(g.out(kn), "K"), (rope_cos, "C"), (rope_sin, "S"), (Pos, "P")], [], [D.NKV, 1, 1],
                   {"HD": D.HD, "NKV": D.NKV, "ROT_HALF": D.ROT_HALF, "MAX_LEN": D.MAX_LEN})
            kv_type = row_major([B, D.NKV * D.MAX_LEN, D.HD], "bf16")
            fa = g.node("fa2_attn",
                        [(g.out(qn), "q"), (g.out(kn), "k"), (vp, "v"), (qp, "qgate"),
                         (g.input(f"{pre}.kv_k_in", kv_type, "state"), "kc_in"),
                         (g.input(f"{pre}.kv_v_in", kv_type, "state"), "vc_in"), (Pos, "P")],
                        [("out", act(D.NH * D.HD)), (f"{pre}.kv_k_new", kv_type, "state"),
                         (f"{pre}.kv_v_new", kv_type, "state")],
                        [D.NH, 1, 1], {"HD": D.HD, "NH": D.NH, "MAX_LEN": D.MAX_LEN, "NKV": D.NKV})
            proj = gemm(g.out(fa), f"{sa}.o_proj.weight", D.H, D.NH * D.HD, False)
        h = residual(proj, h, D.H, "attn")

        normed2 = g.out(g.node("rmsnorm", [(h, "x"), (weight(f"{pre}.post_attention_layernorm.weight", [D.H]), "w")],
                               [("out", act(D.H))], [1, 1, 1], {"N": D.H}))
        gate = gemm(normed2, f"{pre}.mlp.gate_proj.weight", D.INTER, D.H, False)
        up = gemm(normed2, f"{pre}.mlp.up_proj.weight", D.INTER, D.H, False)
        act_ = g.node("swiglu", [(gate, "g"), (up, "u")], [("out", act(D.INTER))], [math.ceil(D.INTER / 1024), 1, 1],
                      {"N": D.INTER})
        down = gemm(g.out(act_), f"{pre}.mlp.down_proj.weight", D.H, D.INTER, False)
        h = residual(down, h, D.H, "mlp")

    fn = g.node("rmsnorm", [(h, "x"), (weight("final.norm.weight", [D.H]), "w")], [("out", act(D.H))], [1, 1, 1],
                {"N": D.H})
    logits = gemm(g.out(fn), "lm_head.weight", D.VOCAB, D.H, False)
    g.node("argmax", [(logits, "logits")],
           [("val", row_major([B], "f32")), ("idx", row_major([B], "i32"))], [1, 1, 1], {"VOCAB": D.VOCAB})
    return g


def expected_node_count(D: Dims = SYNTH) -> int:
    """1 embed + 17 per GDN layer + 19 per full-attention layer + 3 (final norm, lm_head, argmax)."""
    n_fa = sum(1 for l in range(D.NL) if D.is_full_attention(l))
    return 1 + (D.NL - n_fa) * 17 + n_fa * 19 + 3


def with_context(D: Dims, max_len: int) -> Dims:
    return replace(D, MAX_LEN=max_len)
