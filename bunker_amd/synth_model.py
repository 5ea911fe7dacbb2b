"""Random-init weights and decode state for the synthetic Qwen3.5-style model.

Names follow the external tensors of ``model.buildModelGraph``.  Linear weights are Q4_K
(zero-mean, std 1/sqrt(K)), embeddings bf16 N(0,1), norm weights bf16 N(0,0.02) (used as 1+w),
KV caches prefilled with bf16 N(0,1), GDN state f32 N(0,0.02), conv state bf16 N(0,1).

State arrays are returned in the canonical layout (K and V pages both ``[page][kv head][16 tokens]
[HD]``); ``device_state`` converts V pages to the dim-major layout the attention kernel reads.
"""
from __future__ import annotations

import numpy as np

from . import synth
from .model import Dims, L


def rope_tables(D: Dims):
    """cos/sin tables f32 [MAX_LEN, ROT_HALF]: f_i = theta^(-2i/ROT_DIM), evaluated in double
    (prototypes/decode.ts:865-871, prototypes/decode_graph.ts:120-131)."""
    i = np.arange(D.ROT_HALF, dtype=np.float64)
    f = 1.0 / np.power(D.ROPE_THETA, 2.0 * i / D.ROT_DIM)
    ang = np.arange(D.MAX_LEN, dtype=np.float64)[:, None] * f[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def synth_weights(D: Dims, seed: int = 0) -> dict:
    g = synth.rng(seed)
    bf = synth.f32_to_bf16
    W: dict = {}

    def lin(name, N, K):
        W[name] = synth.q4k_centered(g, N, K, 1.0 / np.sqrt(K))

    def norm(name, n):
        W[name] = bf((g.standard_normal(n) * 0.02).astype(np.float32))

    W["embed.weight"] = bf(g.standard_normal((D.VOCAB, D.H), dtype=np.float32))
    for l in range(D.NL):
        p = L(l)
        norm(f"{p}.input_layernorm.weight", D.H)
        norm(f"{p}.post_attention_layernorm.weight", D.H)
        if not D.is_full_attention(l):
            la = f"{p}.linear_attn"
            lin(f"{la}.in_proj_qkv.weight", D.QKVD, D.H)
            lin(f"{la}.in_proj_z.weight", D.ZD, D.H)
            lin(f"{la}.in_proj_a.weight", D.LVH, D.H)
            lin(f"{la}.in_proj_b.weight", D.LVH, D.H)
            lin(f"{la}.out_proj.weight", D.H, D.ZD)
            W[f"{la}.conv1d.weight"] = bf((g.standard_normal((D.QKVD, 4)) * 0.5).astype(np.float32))
            W[f"{la}.A_log"] = (g.standard_normal(D.LVH) * 0.5).astype(np.float32)
            W[f"{la}.dt_bias"] = bf(g.standard_normal(D.LVH).astype(np.float32))
            W[f"{la}.norm.weight"] = (1.0 + 0.02 * g.standard_normal(D.LVD)).astype(np.float32)
        else:
            sa = f"{p}.self_attn"
            lin(f"{sa}.q_proj.weight", D.QGATE, D.H)
            lin(f"{sa}.k_proj.weight", D.KV_DIM, D.H)
            lin(f"{sa}.v_proj.weight", D.KV_DIM, D.H)
            lin(f"{sa}.o_proj.weight", D.H, D.NH * D.HD)
            norm(f"{sa}.q_norm.weight", D.HD)
            norm(f"{sa}.k_norm.weight", D.HD)
        lin(f"{p}.mlp.gate_proj.weight", D.INTER, D.H)
        lin(f"{p}.mlp.up_proj.weight", D.INTER, D.H)
        lin(f"{p}.mlp.down_proj.weight", D.H, D.INTER)
    norm("final.norm.weight", D.H)
    lin("lm_head.weight", D.VOCAB, D.H)
    W["rope_cos"], W["rope_sin"] = rope_tables(D)
    return W


def synth_state(D: Dims, batch: int, seed: int = 1, share_kv_across_batch: bool = False) -> dict:
    """Initial decode state, canonical layout.  KV caches are full of random tokens (the first
    ``pos`` of them are the context; the rest is overwritten as decoding proceeds)."""
    g = synth.rng(seed)
    bf = synth.f32_to_bf16
    S: dict = {}
    pages = D.MAX_LEN // 16
    for l in range(D.NL):
        p = L(l)
        if not D.is_full_attention(l):
            S[f"{p}.conv_state"] = bf(g.standard_normal((batch, 3, D.QKVD), dtype=np.float32))
            S[f"{p}.s_state"] = (g.standard_normal((batch, D.LVH, D.LKD, D.LVD), dtype=np.float32) * np.float32(0.02))
        else:
            nb = 1 if share_kv_across_batch else batch
            for kv in ("kv_k", "kv_v"):
                a = bf(g.standard_normal((nb, pages, D.NKV, 16, D.HD), dtype=np.float32))
                S[f"{p}.{kv}"] = np.broadcast_to(a, (batch, pages, D.NKV, 16, D.HD)) if share_kv_across_batch else a
    return S


def device_state(state: dict) -> dict:
    """Canonical state -> the byte layout of the device buffers (V pages become dim-major)."""
    out = {}
    for k, v in state.items():
        if k.endswith(".kv_v"):
            out[k] = np.ascontiguousarray(np.asarray(v).swapaxes(-1, -2))
        else:
            out[k] = np.ascontiguousarray(v)
    return out
