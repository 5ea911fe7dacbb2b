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

Two chunks are in flight at a time, on two streams with their own activation buffers: what couples them is the
per-layer state (conv rows and S, or the KV cache), so chunk c+1 waits at each layer's state-touching op for the
event chunk c recorded behind its own.  The GDN scan keeps a quarter of the SIMDs busy with one wave each; the other
chunk's matmuls run beside it.
"""
from __future__ import annotations

from typing import Callable, Sequence

import numpy as np

from . import runtime as rt
from .model import Dims, L
from . import runner as _runner
from .runner import DecodeEnv, Q8OUT_MIN_BATCH


class _Slot:
    """Activation buffers, kernel handles (they own their workspaces) and the stream of one chunk in flight."""

    def __init__(self, owner: "Prefill", stream):
        D, T = owner.D, owner.chunk
        self.stream = stream
        self.buf = {name: owner._alloc(T * n * b) for name, (n, b) in {
            "x": (D.H, 2), "h": (D.H, 2), "qkv": (D.QKVD, 2), "z": (D.ZD, 2), "a": (D.LVH, 4), "b": (D.LVH, 4),
            "conv": (D.QKVD, 2), "mix": (max(D.ZD, D.NH * D.HD), 2), "qg": (D.QGATE, 2), "k": (D.KV_DIM, 2), "v": (D.KV_DIM, 2),
            "act": (D.INTER, 2), "act_q8": (D.INTER // 32 * 36, 1)}.items()}
        self.kernels: dict[int, dict] = {}
        self.done = [rt.Event() for _ in range(D.NL)]        # layer l's state of this slot's chunk has been written


class Prefill:
    def __init__(self, D: Dims, env: DecodeEnv, chunk: int = 1024, on_attention: Callable | None = None, overlap: bool | int = True,
                 gdn_chunked: bool = False, attn_exact: bool = True):
        """``env`` supplies the weights and the state buffers (those of sequence ``seq`` are updated in place).
        ``on_attention(layer, first_token_index, rows)`` receives each full-attention layer's output
        (uint16 bf16 bits ``[T, NH*HD]``) as it is produced — for tests.  ``overlap``: chunks in flight (True = 2,
        False = 1: everything on the library's first stream).  ``gdn_chunked``: the Gated-DeltaNet recurrence in chunks of
        64 tokens on the f32 matrix instruction (the form of the reference's prefill prototypes) instead of the scan;
        state and outputs then agree with T decode steps to ~1e-6 relative, not to the bit.  ``attn_exact=False``: the
        causal attention of a chunk on the bf16 matrix cores (within 2e-2) instead of the double-precision decode kernel."""
        if chunk < 1 or chunk > 4096:
            raise ValueError("Prefill: chunk must be 1..4096 tokens")
        self.D, self.env, self.chunk, self.on_attention = D, env, int(chunk), on_attention
        self.gdn_chunked = bool(gdn_chunked)
        self.attn_exact = bool(attn_exact)       # double-precision attention (the bits of T decode steps), or the tiled matrix-instruction form
        self._owned: list[int] = []
        in_flight = 2 if overlap is True else max(int(overlap), 1)
        self._streams = [rt.Stream() for _ in range(in_flight)] if in_flight > 1 else []
        self.slots = [_Slot(self, st) for st in (self._streams or [None])]
        self.d_table = self._alloc(max(D.MAX_LEN // 16, 1) * 4)
        self.d_ids = self._alloc(D.MAX_LEN * 4)          # token ids and positions of the whole prompt, uploaded once per run
        self.d_pos = self._alloc(D.MAX_LEN * 4)
        self.d_logits = self._alloc(D.VOCAB * 4)
        self.d_val = self._alloc(4)
        self.d_idx = self._alloc(4)
        self.k_head = rt.compileAndLoad(f"gemv_fused K={D.H} pro=2 G=1 N0={D.VOCAB} epi0=0")
        self.k_argmax = rt.compileAndLoad(f"argmax VOCAB={D.VOCAB}")

    @property
    def buf(self) -> dict:
        """Activation buffers of the first slot (the only one when ``overlap=False``)."""
        return self.slots[0].buf

    def _alloc(self, nbytes: int) -> int:
        p = rt.cuAlloc(max(int(nbytes), 16))
        self._owned.append(p)
        return p

    def close(self) -> None:
        rt.cuSync()
        for p in self._owned:
            rt.cuFree(p)
        self._owned = []
        for sl in self.slots:
            for ev in sl.done:
                ev.destroy()
        for st in self._streams:
            st.destroy()
        self._streams, self.slots = [], []

    def _kernels(self, slot: "_Slot", T: int) -> dict:
        """Kernel handles of a slot for a run of T tokens (the specs carry T; handles own their workspaces)."""
        if T in slot.kernels:
            return slot.kernels[T]
        D = self.D
        bp = f" batch={T}" if T != 1 else ""
        c = rt.compileAndLoad
        k = {
            "embed": c(f"embed H={D.H} VOCAB={D.VOCAB} ids_dev=1" + bp),
            "gdn_in": c(f"gemv_fused K={D.H} pro=2 G=4 N0={D.QKVD} epi0=1 N1={D.ZD} epi1=1 N2={D.LVH} epi2=0 N3={D.LVH} epi3=0" + bp),
            "conv": c(f"conv1d_prefill QKVD={D.QKVD} T={T}"),
            "gdn": c(f"gdn_prefill LVH={D.LVH} T={T}" + (" chunked=1" if self.gdn_chunked else "")),
            "gdn_out": c(f"gemv_fused K={D.ZD} pro=1 G=1 N0={D.H} epi0=2" + bp),
            "fa_in": c(f"gemv_fused K={D.H} pro=2 G=3 N0={D.QGATE} epi0=1 N1={D.KV_DIM} epi1=1 N2={D.KV_DIM} epi2=1" + bp),
            "fa": c(f"fa2_prefill HD={D.HD} NH={D.NH} NKV={D.NKV} MAX_LEN={D.MAX_LEN} ROT_HALF={D.ROT_HALF} T={T}"
                    + ("" if self.attn_exact else " exact=0")),
            "fa_out": c(f"gemv_fused K={D.NH * D.HD} pro=1 G=1 N0={D.H} epi0=2" + bp),
        }
        # batched form: the matmul leaves the SwiGLU result as Q8_1 blocks too and the down projection reads those
        self_q8 = T >= Q8OUT_MIN_BATCH and D.INTER % 32 == 0
        k["mlp_q8"] = self_q8
        k["mlp_in"] = c(f"gemv_fused K={D.H} pro=2 G=2 swiglu=1 N0={D.INTER} N1={D.INTER}" + bp + (" q8out=1" if self_q8 else ""))
        k["mlp_out"] = c(f"gemv_fused K={D.INTER} pro={0 if self_q8 else 1} G=1 N0={D.H} epi0=2" + bp)
        slot.kernels[T] = k
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
        D, e = self.D, self.env
        tokens = np.asarray(tokens, np.int32).ravel()
        n = tokens.size
        if n < 1:
            raise ValueError("Prefill.run: empty prompt")
        if pos0 < 0 or pos0 + n > D.MAX_LEN:
            raise ValueError(f"Prefill.run: positions {pos0}..{pos0 + n - 1} exceed MAX_LEN={D.MAX_LEN}")
        ppseq = D.MAX_LEN // 16
        rt.cuHtoD(self.d_table, (seq * ppseq + np.arange(ppseq, dtype=np.int32)))
        rt.cuHtoD(self.d_ids, np.ascontiguousarray(tokens))
        rt.cuHtoD(self.d_pos, (pos0 + np.arange(n, dtype=np.int32)))
        start = rt.Event().record()          # the uploads (and whatever the caller queued before) precede both streams
        prev: _Slot | None = None            # the slot that holds the chunk before this one
        done = 0
        ci = 0
        while done < n:
            T = min(self.chunk, n - done)
            slot = self.slots[ci % len(self.slots)]
            if slot.stream is not None:
                slot.stream.__enter__()
            try:
                if ci < len(self.slots) and slot.stream is not None:
                    rt.streamWaitEvent(start)
                self._chunk(slot, prev if prev is not slot else None, T, seq, done)
            finally:
                if slot.stream is not None:
                    slot.stream.__exit__(None, None, None)
            prev, last_T = slot, T
            done += T
            ci += 1
        # the last prompt token's row: final norm + lm_head + argmax, behind the last chunk on its stream
        if prev.stream is not None:
            prev.stream.__enter__()
        try:
            W = e.ptr
            last = prev.buf["x"] + (last_T - 1) * D.H * 2
            self._launch(self.k_head, [last, W["final.norm.weight"], W["lm_head.weight"], self.d_logits], "lm_head")
            self._launch(self.k_argmax, [self.d_logits, self.d_val, self.d_idx], "argmax")
        finally:
            if prev.stream is not None:
                prev.stream.__exit__(None, None, None)
        rt.cuSync()
        start.destroy()
        tok = rt.from_device(self.d_idx, (1,), np.int32)
        val = rt.from_device(self.d_val, (1,), np.float32)
        return int(tok[0]), float(val[0])

    def _chunk(self, slot: "_Slot", prev: "_Slot | None", T: int, seq: int, first_index: int) -> None:
        """Queue the T tokens from ``first_index`` on, on the selected stream.  ``prev`` holds the chunk before them on
        another stream: each layer's state-touching ops wait for that chunk's event of the same layer and record this
        slot's own behind them."""
        D, e, B = self.D, self.env, slot.buf
        k = self._kernels(slot, T)
        W = e.ptr
        d_ids, d_pos = self.d_ids + 4 * first_index, self.d_pos + 4 * first_index
        self._launch(k["embed"], [W["embed.weight"], d_ids, B["x"]], "embed")
        x, h = B["x"], B["h"]
        for layer in range(D.NL):
            p = L(layer)
            if not D.is_full_attention(layer):
                la = f"{p}.linear_attn"
                self._launch(k["gdn_in"], [x, W[f"{p}.input_layernorm.weight"], W[f"{la}.in_proj_qkv.weight"], B["qkv"],
                                           W[f"{la}.in_proj_z.weight"], B["z"], W[f"{la}.in_proj_a.weight"], B["a"],
                                           W[f"{la}.in_proj_b.weight"], B["b"]], f"{p} in_proj")
                if prev is not None:
                    rt.streamWaitEvent(prev.done[layer])
                cs = self._state(f"{p}.conv_state", 3 * D.QKVD * 2, seq)
                self._launch(k["conv"], [B["qkv"], cs, W[f"{la}.conv1d.weight"], B["conv"], cs], f"{p} conv1d")
                ss = self._state(f"{p}.s_state", D.LVH * D.LKD * D.LVD * 4, seq)
                self._launch(k["gdn"], [B["conv"], B["z"], W[f"{la}.A_log"], W[f"{la}.dt_bias"], B["a"], B["b"],
                                        W[f"{la}.norm.weight"], ss, B["mix"], ss], f"{p} gdn")
                slot.done[layer].record()
                self._launch(k["gdn_out"], [B["mix"], W[f"{la}.out_proj.weight"], x, h], f"{p} out_proj")
            else:
                sa = f"{p}.self_attn"
                self._launch(k["fa_in"], [x, W[f"{p}.input_layernorm.weight"], W[f"{sa}.q_proj.weight"], B["qg"],
                                          W[f"{sa}.k_proj.weight"], B["k"], W[f"{sa}.v_proj.weight"], B["v"]], f"{p} qkv")
                if prev is not None:
                    rt.streamWaitEvent(prev.done[layer])
                kc = e.state_bufs[f"{p}.kv_k"][0]
                vc = e.state_bufs[f"{p}.kv_v"][0]
                self._launch(k["fa"], [B["qg"], B["k"], B["v"], W[f"{sa}.q_norm.weight"], W[f"{sa}.k_norm.weight"],
                                       W["rope_cos"], W["rope_sin"], d_pos, self.d_table, kc, vc, B["mix"]], f"{p} attention")
                slot.done[layer].record()
                if self.on_attention is not None:
                    rt.cuSync()
                    self.on_attention(layer, first_index, rt.from_device(B["mix"], (T, D.NH * D.HD), np.uint16))
                self._launch(k["fa_out"], [B["mix"], W[f"{sa}.o_proj.weight"], x, h], f"{p} o_proj")
            self._launch(k["mlp_in"], [h, W[f"{p}.post_attention_layernorm.weight"], W[f"{p}.mlp.gate_proj.weight"],
                                       W[f"{p}.mlp.up_proj.weight"], B["act"]] + ([B["act_q8"]] if k["mlp_q8"] else []), f"{p} gate/up")
            self._launch(k["mlp_out"], [B["act_q8"] if k["mlp_q8"] else B["act"], W[f"{p}.mlp.down_proj.weight"], h, x], f"{p} down")
