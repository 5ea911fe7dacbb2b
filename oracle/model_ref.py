"""CPU restatement of one decode step of the model graph, op by op, on the oracle's C ops.

TEST INFRASTRUCTURE ONLY (see oracle.c).  Written as straight-line code in the node order of
src/model.ts:46-204, independently of the product's graph/runner: embed -> per layer
[rmsnorm -> (GDN: qkv, z, conv1d, a, b, gdn, out_proj | FA: q, k, v, qnorm, rope, knorm,
ropek, fa2_attn, o_proj) -> cast -> add -> rmsnorm -> gate, up, swiglu, down -> cast -> add]
-> rmsnorm -> lm_head -> argmax.  Every matmul is "quantize the bf16 activation to Q8_1,
Q4_K x Q8_1 dot" (bench/bench.ts:10-72 on 144-byte super-blocks), accumulated in double.

Weights are the dict of ``bunker_amd.synth_model.synth_weights`` (plain numpy byte arrays),
state is the canonical layout of ``synth_state`` and is updated in place.
"""
from __future__ import annotations

import numpy as np

from . import oracle as orc


def _L(l):
    return f"model.layers.{l}"


class RefModel:
    def __init__(self, D, weights: dict, state: dict, batch: int = 1):
        self.D, self.W, self.B = D, weights, batch
        self.S = {k: np.array(v, copy=True) for k, v in state.items()}
        self.margins = []        # top-1 minus top-2 logit of every (step, sequence)
        self.trace = None        # set to a list to record (op, output array) in node order of one step
        self.attn_err = []       # max |own attention - injected attention| per injected layer call

    def _t(self, op, arr):
        if self.trace is not None:
            self.trace.append((op, None if arr is None else np.array(arr, copy=True)))
        return arr

    def gemm(self, a_bf16, wname, N, K, cast):
        xq = orc.pack_q8_1(orc.bf16_to_f32(a_bf16))
        y = orc.gemv_q4k_q8_1(self.W[wname], xq, N, K, acc64=True)
        return self._t("gemm", orc.cast_bf16(y) if cast else y)

    def step_one(self, b: int, token: int, pos: int, attn_override: dict | None = None):
        D, W, S = self.D, self.W, self.S
        t = self._t
        h = t("embed", orc.embed(W["embed.weight"], token, D.H))
        for l in range(D.NL):
            p = _L(l)
            normed = t("rmsnorm", orc.rmsnorm(h, W[f"{p}.input_layernorm.weight"]))
            if not D.is_full_attention(l):
                la = f"{p}.linear_attn"
                qkv = self.gemm(normed, f"{la}.in_proj_qkv.weight", D.QKVD, D.H, True)
                z = self.gemm(normed, f"{la}.in_proj_z.weight", D.ZD, D.H, True)
                conv, st_new = orc.conv1d_decode(qkv, S[f"{p}.conv_state"][b], W[f"{la}.conv1d.weight"])
                S[f"{p}.conv_state"][b] = st_new
                t("conv1d_decode", conv)
                a_p = self.gemm(normed, f"{la}.in_proj_a.weight", D.LVH, D.H, False)
                b_p = self.gemm(normed, f"{la}.in_proj_b.weight", D.LVH, D.H, False)
                out, S_new = orc.gdn_step(conv, z, W[f"{la}.A_log"], W[f"{la}.dt_bias"], a_p, b_p, W[f"{la}.norm.weight"],
                                          S[f"{p}.s_state"][b], D.LVH, D.LKD, D.LVD)
                S[f"{p}.s_state"][b] = S_new
                t("gdn_delta_rule", out)
                proj = self.gemm(out, f"{la}.out_proj.weight", D.H, D.ZD, False)
            else:
                sa = f"{p}.self_attn"
                qp = self.gemm(normed, f"{sa}.q_proj.weight", D.QGATE, D.H, True)
                kp = self.gemm(normed, f"{sa}.k_proj.weight", D.KV_DIM, D.H, True)
                vp = self.gemm(normed, f"{sa}.v_proj.weight", D.KV_DIM, D.H, True)
                qn = orc.headnorm(qp, W[f"{sa}.q_norm.weight"], D.NH, D.HD, 2 * D.HD)
                qn = t("qnorm", orc.rope(qn, W["rope_cos"], W["rope_sin"], pos, D.NH, D.HD, D.ROT_HALF))   # after rope
                t("rope", None)
                kn = orc.headnorm(kp, W[f"{sa}.k_norm.weight"], D.NKV, D.HD, D.HD)
                kn = t("knorm", orc.rope(kn, W["rope_cos"], W["rope_sin"], pos, D.NKV, D.HD, D.ROT_HALF))
                t("ropek", None)
                kc, vc = S[f"{p}.kv_k"][b], S[f"{p}.kv_v"][b]          # [pages, NKV, 16, HD] views, written in place
                bt = np.arange(kc.shape[0], dtype=np.int32)
                orc.kv_append(kn, vp, kc, vc, bt, pos, D.NKV, D.HD, 16)
                att, _ = orc.attn_decode_paged(qn, kc, vc, bt[None], np.array([pos + 1], np.int32), 1, D.NH, D.NKV, D.HD, 16,
                                               gate=qp[D.HD:], gate_bstride=0, gate_hstride=2 * D.HD)
                if attn_override is not None:
                    # continue from the attention output of the implementation under test (bf16 [NH*HD]);
                    # the checker's own result stays the yardstick for that output's tolerance
                    inj = np.ascontiguousarray(attn_override[l], np.uint16).reshape(att.shape)
                    self.attn_err.append(float(np.abs(orc.bf16_to_f32(inj).astype(np.float64) - orc.bf16_to_f32(att)).max()))
                    att = inj
                t("fa2_attn", att.ravel())
                proj = self.gemm(att.ravel(), f"{sa}.o_proj.weight", D.H, D.NH * D.HD, False)
            h = t("add", orc.add_bf16(t("cast", orc.cast_bf16(proj)), h))
            normed2 = t("rmsnorm", orc.rmsnorm(h, W[f"{p}.post_attention_layernorm.weight"]))
            gate = self.gemm(normed2, f"{p}.mlp.gate_proj.weight", D.INTER, D.H, False)
            up = self.gemm(normed2, f"{p}.mlp.up_proj.weight", D.INTER, D.H, False)
            act = t("swiglu", orc.swiglu(gate, up))
            down = self.gemm(act, f"{p}.mlp.down_proj.weight", D.H, D.INTER, False)
            h = t("add", orc.add_bf16(h, t("cast", orc.cast_bf16(down))))
        fn = t("rmsnorm", orc.rmsnorm(h, W["final.norm.weight"]))
        logits = self.gemm(fn, "lm_head.weight", D.VOCAB, D.H, False)
        val, idx = orc.argmax(logits)
        return idx, val, logits

    def step(self, tokens, pos, attn_override: dict | None = None):
        """One token for every sequence; returns (idx int32 [B], val f32 [B], logits f32 [B, V]).

        attn_override: {layer: bf16 [B, NH*HD]} replaces the attention outputs of those layers."""
        out_i, out_v, out_l = [], [], []
        marg = []
        for b in range(self.B):
            if not self.S:
                raise RuntimeError("no state")
            ov = None if attn_override is None else {l: a[b] for l, a in attn_override.items()}
            i, v, lg = self.step_one(b, int(tokens[b]), int(pos[b]), ov)
            out_i.append(i); out_v.append(v); out_l.append(lg)
            top2 = np.partition(lg, -2)[-2:]
            marg.append(float(top2[1] - top2[0]))
        self.margins.append(marg)
        return np.array(out_i, np.int32), np.array(out_v, np.float32), np.stack(out_l)

    def decode(self, start_tokens, start_pos, steps: int):
        toks = np.asarray(start_tokens, np.int32).reshape(self.B).copy()
        pos = np.broadcast_to(np.asarray(start_pos, np.int32), (self.B,)).copy()
        hist_t, hist_v = [], []
        for _ in range(steps):
            idx, val, _ = self.step(toks, pos)
            hist_t.append(idx); hist_v.append(val)
            toks, pos = idx, pos + 1
        return np.stack(hist_t), np.stack(hist_v)


def free_run_report(got_tokens, got_vals, ref_tokens, ref_vals, margins) -> dict:
    """Two independent greedy decodes side by side: ``got`` from the implementation under test, ``ref`` and the
    top-1/top-2 ``margins`` from ``RefModel.decode``.  Arrays are [steps, sequences].

    A sequence is compared up to its first differing token (afterwards the two runs decode different texts).
    ``noise`` is |winning logit of the implementation - winning logit of the checker| on the compared steps."""
    got_tokens, ref_tokens = np.asarray(got_tokens), np.asarray(ref_tokens)
    margins = np.asarray(margins, np.float64).reshape(ref_tokens.shape)
    noise = np.abs(np.asarray(got_vals, np.float64) - np.asarray(ref_vals, np.float64))
    steps, nseq = ref_tokens.shape
    matched, first_div, worst = 0, None, None
    max_noise, min_margin = 0.0, float("inf")
    for b in range(nseq):
        for s in range(steps):
            if got_tokens[s, b] != ref_tokens[s, b]:
                seen = float(noise[:s, b].max()) if s else 0.0
                if first_div is None or s < first_div["step"]:
                    first_div = {"step": s, "sequence": b, "margin": float(margins[s, b]), "noise_before": seen}
                break
            matched += 1
            max_noise = max(max_noise, float(noise[s, b]))
            min_margin = min(min_margin, float(margins[s, b]))
    return {"argmax_match": f"{matched}/{steps * nseq}", "matched": matched, "compared": steps * nseq, "steps": steps,
            "sequences": nseq, "first_divergence": first_div,
            "min_margin_on_matched_steps": None if min_margin == float("inf") else round(min_margin, 6),
            "max_logit_noise_on_matched_steps": round(max_noise, 6)}
