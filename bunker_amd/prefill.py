"""Prompt processing for the decode step: T tokens of one sequence at a time through every layer, leaving the
recurrent state (conv rows, GDN S), the KV cache and the first generated token exactly as T single-token steps
would (the reference's own prefill is prototype-level: prototypes/qwen35.ts:261-400 runs the layers with
M = seq matmuls, prototypes/fa2_vllm.ts and prototypes/gdn_fast.ts hold the attention and GDN prototypes).

Rows of every activation buffer are tokens.  Per layer the launches mirror the fused decode groups of
``runner.fusedPartition`` with ``batch = T`` (the matmuls then run on the int8 matrix cores), and the three ops
that couple the tokens of a sequence use their run forms: ``conv1d_prefill``, ``gdn_prefill`` (state in
registers for the whole run), ``fa2_prefill`` (cache append for all T tokens, then causal attention).  A prompt
longer than ``chunk`` tokens is processed in chunks; the state carries over.

Everything except attention follows the arithmetic rules of the single-token kernels, so the state and the
logits of the last prompt token equal those of a token-by-token run bit for bit wherever attention outputs do.
"""
from __future__ import annotations

from typing import Callable, Sequence

import numpy as np

from . import runtime as rt
from .model import Dims, L
from .runner import DecodeEnv


class Prefill:
    def __init__(self, D: Dims, env: DecodeEnv, chunk: int = 1024, on_attention: Callable | None = None):
        """``env`` supplies the weights and the state buffers (those of sequence ``seq`` are updated in place).
        ``on_attention(layer, first_token_index, rows)`` receives each full-attention layer's output
        (uint16 bf16 bits ``[T, NH*HD]``) as it is produced — for tests."""
        if chunk < 1 or chunk > 4096:
            raise ValueError("Prefill: chunk must be 1..4096 tokens")
        self.D, self.env, self.chunk, self.on_attention = D, env, int(chunk), on_attention
        self._k: dict[int, dict] = {}
        self._owned: list[int] = []
        T = self.chunk
        self.buf = {name: self._alloc(T * n * b) for name, (n, b) in {
            "x": (D.H, 2), "h": (D.H, 2), "qkv": (D.QKVD, 2), "z": (D.ZD, 2), "a": (D.LVH, 4), "b": (D.LVH, 4),
            "conv": (D.QKVD, 2), "mix": (max(D.ZD, D.NH * D.HD), 2), "qg": (D.QGATE, 2), "k": (D.KV_DIM, 2), "v": (D.KV_DIM, 2),
            "act": (D.INTER, 2)}.items()}
        self.d_ids = self._alloc(T * 4)
        self.d_pos = self._alloc(T * 4)
        self.d_table = self._alloc(max(D.MAX_LEN // 16, 1) * 4)
        self.d_logits = self._alloc(D.VOCAB * 4)
        self.d_val = self._alloc(4)
        self.d_idx = self._alloc(4)
        self.k_head = rt.compileAndLoad(f"gemv_fused K={D.H} pro=2 G=1 N0={D.VOCAB} epi0=0")
        self.k_argmax = rt.compileAndLoad(f"argmax VOCAB={D.VOCAB}")

    def _alloc(self, nbytes: int) -> int:
        p = rt.cuAlloc(max(int(nbytes), 16))
        self._owned.append(p)
        return p

    def close(self) -> None:
        for p in self._owned:
            rt.cuFree(p)
        self._owned = []

    def _kernels(self, T: int) -> dict:
        """Kernel handles for a run of T tokens (the specs carry T; handles own their workspaces)."""
        if T in self._k:
            return self._k[T]
        D = self.D
        bp = f" batch={T}" if T != 1 else ""
        c = rt.compileAndLoad
        k = {
            "embed": c(f"embed H={D.H} VOCAB={D.VOCAB} ids_dev=1" + bp),
            "gdn_in": c(f"gemv_fused K={D.H} pro=2 G=4 N0={D.QKVD} epi0=1 N1={D.ZD} epi1=1 N2={D.LVH} epi2=0 N3={D.LVH} epi3=0" + bp),
            "conv": c(f"conv1d_prefill QKVD={D.QKVD} T={T}"),
            "gdn": c(f"gdn_prefill LVH={D.LVH} T={T}"),
            "gdn_out": c(f"gemv_fused K={D.ZD} pro=1 G=1 N0={D.H} epi0=2" + bp),
            "fa_in": c(f"gemv_fused K={D.H} pro=2 G=3 N0={D.QGATE} epi0=1 N1={D.KV_DIM} epi1=1 N2={D.KV_DIM} epi2=1" + bp),
            "fa": c(f"fa2_prefill HD={D.HD} NH={D.NH} NKV={D.NKV} MAX_LEN={D.MAX_LEN} ROT_HALF={D.ROT_HALF} T={T}"),
            "fa_out": c(f"gemv_fused K={D.NH * D.HD} pro=1 G=1 N0={D.H} epi0=2" + bp),
            "mlp_in": c(f"gemv_fused K={D.H} pro=2 G=2 swiglu=1 N0={D.INTER} N1={D.INTER}" + bp),
            "mlp_out": c(f"gemv_fused K={D.INTER} pro=1 G=1 N0={D.H} epi0=2" + bp),
        }
        self._k[T] = k
        return k

    def _launch(self, k, args, what: str) -> None:
        rc = rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], args)
        if rc != 0:
            raise rt.BunkerError(f"prefill {what}: {rt.last_error()} (rc={rc})")

    def _state(self, key: str, row_bytes: int, seq: int) -> int:
        e = self.env
        return e.state_bufs[key][e.state_cur[key]] + seq * row_bytes

    def run(self, tokens: Sequence[int], seq: int = 0, pos0: int = 0):
        """Feed ``tokens`` at positions pos0.. of sequence ``seq``; returns (next token id, its logit).
        The logits of the last prompt token stay in ``self.d_logits`` (f32 [VOCAB])."""
        D, e, B = self.D, self.env, self.buf
        tokens = np.asarray(tokens, np.int32).ravel()
        n = tokens.size
        if n < 1:
            raise ValueError("Prefill.run: empty prompt")
        if pos0 < 0 or pos0 + n > D.MAX_LEN:
            raise ValueError(f"Prefill.run: positions {pos0}..{pos0 + n - 1} exceed MAX_LEN={D.MAX_LEN}")
        ppseq = D.MAX_LEN // 16
        rt.cuHtoD(self.d_table, (seq * ppseq + np.arange(ppseq, dtype=np.int32)))
        W = e.ptr
        done = 0
        last_T = 0
        while done < n:
            T = min(self.chunk, n - done)
            last_T = T
            k = self._kernels(T)
            rt.cuHtoD(self.d_ids, np.ascontiguousarray(tokens[done:done + T]))
            rt.cuHtoD(self.d_pos, (pos0 + done + np.arange(T, dtype=np.int32)))
            self._launch(k["embed"], [W["embed.weight"], self.d_ids, B["x"]], "embed")
            x, h = B["x"], B["h"]
            for layer in range(D.NL):
                p = L(layer)
                if not D.is_full_attention(layer):
                    la = f"{p}.linear_attn"
                    self._launch(k["gdn_in"], [x, W[f"{p}.input_layernorm.weight"], W[f"{la}.in_proj_qkv.weight"], B["qkv"],
                                               W[f"{la}.in_proj_z.weight"], B["z"], W[f"{la}.in_proj_a.weight"], B["a"],
                                               W[f"{la}.in_proj_b.weight"], B["b"]], f"{p} in_proj")
                    cs = self._state(f"{p}.conv_state", 3 * D.QKVD * 2, seq)
                    self._launch(k["conv"], [B["qkv"], cs, W[f"{la}.conv1d.weight"], B["conv"], cs], f"{p} conv1d")
                    ss = self._state(f"{p}.s_state", D.LVH * D.LKD * D.LVD * 4, seq)
                    self._launch(k["gdn"], [B["conv"], B["z"], W[f"{la}.A_log"], W[f"{la}.dt_bias"], B["a"], B["b"],
                                            W[f"{la}.norm.weight"], ss, B["mix"], ss], f"{p} gdn")
                    self._launch(k["gdn_out"], [B["mix"], W[f"{la}.out_proj.weight"], x, h], f"{p} out_proj")
                else:
                    sa = f"{p}.self_attn"
                    self._launch(k["fa_in"], [x, W[f"{p}.input_layernorm.weight"], W[f"{sa}.q_proj.weight"], B["qg"],
                                              W[f"{sa}.k_proj.weight"], B["k"], W[f"{sa}.v_proj.weight"], B["v"]], f"{p} qkv")
                    kc = e.state_bufs[f"{p}.kv_k"][0]
                    vc = e.state_bufs[f"{p}.kv_v"][0]
                    self._launch(k["fa"], [B["qg"], B["k"], B["v"], W[f"{sa}.q_norm.weight"], W[f"{sa}.k_norm.weight"],
                                           W["rope_cos"], W["rope_sin"], self.d_pos, self.d_table, kc, vc, B["mix"]], f"{p} attention")
                    if self.on_attention is not None:
                        rt.cuSync()
                        self.on_attention(layer, done, rt.from_device(B["mix"], (T, D.NH * D.HD), np.uint16))
                    self._launch(k["fa_out"], [B["mix"], W[f"{sa}.o_proj.weight"], x, h], f"{p} o_proj")
                self._launch(k["mlp_in"], [h, W[f"{p}.post_attention_layernorm.weight"], W[f"{p}.mlp.gate_proj.weight"],
                                           W[f"{p}.mlp.up_proj.weight"], B["act"]], f"{p} gate/up")
                self._launch(k["mlp_out"], [B["act"], W[f"{p}.mlp.down_proj.weight"], h, x], f"{p} down")
            done += T
        # the last prompt token's row: final norm + lm_head + argmax
        last = B["x"] + (last_T - 1) * D.H * 2
        self._launch(self.k_head, [last, W["final.norm.weight"], W["lm_head.weight"], self.d_logits], "lm_head")
        self._launch(self.k_argmax, [self.d_logits, self.d_val, self.d_idx], "argmax")
        rt.cuSync()
        tok = rt.from_device(self.d_idx, (1,), np.int32)
        val = rt.from_device(self.d_val, (1,), np.float32)
        return int(tok[0]), float(val[0])
