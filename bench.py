#!/usr/bin/env python3
"""Benchmark of the decode hot path on one MI355X.

Headline workload (BASELINE.json configs[1]): the Q4_K x Q8_1 GEMV at the four decode
shapes, batch 1 — qkv 2048->6144, gate+up 2048->12288, down 6144->2048, lm_head
2048->151936.  One "step" is one launch of each shape.  Weights are resident in HBM before
timing and every launch of a shape reads a different copy out of a >= 600 MB rotation of that
shape, so neither L2 nor the 256 MiB Infinity Cache serves re-reads.  `value` is algorithmic
GB/s over the whole timed region (formula: N*K*144/256 + (K/32)*36 + N*4 bytes per launch).

The timed region holds exactly K steps, grouped by shape: W warm-up launches of the shape, a
HIP event, its K launches (replayed from one HIP graph, or queued from the host with
--mode stream), a HIP event (both on the library's stream).  That gives each kernel's average
launch duration from the same region that `value` is taken from.

Further sections, reported under "decode" and "kernels" of the same line: greedy decode of the
synthetic Qwen3.5-style model (BASELINE configs[4]) at batch 1 and 32 in tok/s against the
byte floor of one step, and the gated-DeltaNet step (configs[2]) and the paged decode attention
(configs[3]) in algorithmic GB/s, and under "gemm_bs32" the batch-32 int8-MFMA matmul at the
decode shapes (weight GB/s and int8 TOP/s).  `--sections gemv` runs the headline part alone.

Prints ONE JSON line.  `python bench.py --gpus 1 --steps 2000 --warmup 500`.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of every profiled kernel, from rocprofv3 --pmc runs (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch,
# each scaled by what the same counter reads for a plain copy of known size).  One line per kernel and shape:
# `kernel | shape | traffic bytes per launch | algorithmic bytes per launch`; the summaries beside it give the commands.
TRAFFIC_TABLE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic_per_launch.txt")


def measured_traffic(kernel: str, shape: str):
    """Measured HBM bytes per launch of `kernel` at `shape`, or None when no counter run covers that pair."""
    try:
        with open(TRAFFIC_TABLE) as f:
            for line in f:
                cols = [c.strip() for c in line.split("|")]
                if len(cols) >= 4 and not line.startswith("#") and cols[0].replace(" ", "") == kernel.replace(" ", "") and cols[1] == shape:
                    return int(cols[2])
    except OSError:
        pass
    return None
SHAPES = [("qkv", 6144, 2048), ("gate_up", 12288, 2048), ("down", 2048, 6144), ("lm_head", 151936, 2048)]
ROTATION_BYTES = 600e6  # every shape rotates through copies of its matrix that add up to at least this much
PREWARM_S = 0.4         # untimed GEMV launches in front of the timed region (clock warm-up; reported as prewarm_ms)


def gemv_bytes(N, K, batch=1):
    return N * K * 144 // 256 + batch * (K // 32) * 36 + batch * N * 4


def _host_info():
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return {"cpu_model": model, "os_cpu_count": os.cpu_count(), "usable_cpus": usable}


def _timed(fn, seconds, max_reps=1_000_000):
    """Repeat fn() for about `seconds`; returns (repetitions, elapsed seconds)."""
    fn()
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        dt = time.perf_counter() - t0
        if dt > seconds or reps >= max_reps:
            return reps, dt


def cpu_baseline(decode_inputs=None, seconds_per_op=1.5):
    """The CPU restatement of the path's ops (the C oracle: the reference's host loops of bench/bench.ts:10-72,
    prototypes/gdn_gated.ts:67-88, prototypes/fa2_vllm.ts:114-139) timed on this machine's host cores, on bounded samples
    of the workload: one decode shape or one configuration per op, about `seconds_per_op` seconds each.  A reported
    baseline, not a target.  The full decode step of the checker is timed on the same run that compares its tokens with the GPU's."""
    from oracle import oracle as orc
    from bunker_amd import synth

    orc.build()
    host = _host_info()
    # all-core legs use the CPUs this process may run on, capped by OMP_NUM_THREADS when the machine sets it
    all_threads = host["usable_cpus"]
    if os.environ.get("OMP_NUM_THREADS", "").isdigit():
        all_threads = min(all_threads, int(os.environ["OMP_NUM_THREADS"]))
    host["threads_all_core_legs"] = all_threads
    bf = synth.f32_to_bf16
    g = synth.rng(1)
    ops = {}

    # Q8_1 quantizer (packQ8_1, bench/bench.ts:53-72): scalar loop, one thread
    K = 6144
    x = g.standard_normal(K * 64).astype(np.float32)            # 64 activation rows of the down projection
    orc.set_threads(1)
    reps, dt = _timed(lambda: orc.pack_q8_1(x), seconds_per_op)
    ops["quantize_q8_1"] = {"threads": 1, "value": round(reps * x.size / dt / 1e6, 1), "unit": "M elements/s",
                            "GBps_in": round(reps * x.nbytes / dt / 1e9, 3), "sample": f"{reps} x {x.size} f32 values in {dt:.1f} s"}

    # Q4_K x Q8_1 GEMV (qmm, bench/bench.ts:10-38 on super-blocks): gate_up shape, one thread and all cores
    name, N, K = SHAPES[1]
    W = synth.q4k_random(g, N, K)
    xq = orc.pack_q8_1(g.standard_normal(K).astype(np.float32))
    gemv = {}
    for label, th in (("1_thread", 1), ("all_cores", all_threads)):
        orc.set_threads(th)
        reps, dt = _timed(lambda: orc.gemv_q4k_q8_1(W, xq, N, K, acc64=False), seconds_per_op * (2 if th > 1 else 1))
        gemv[label] = {"threads": th, "value": round(reps * gemv_bytes(N, K) / dt / 1e9, 3), "unit": "GB/s",
                       "sample": f"{reps} x {name} GEMV (N={N}, K={K}, batch 1) in {dt:.1f} s"}
    ops["gemv_q4k_q8_1"] = gemv
    del W

    # gated-DeltaNet step (refGDN, prototypes/gdn_gated.ts:67-88 at T=1): BASELINE configs[2], batch 1, 32 heads
    Hg = 32
    S = (g.standard_normal((Hg, 128, 128), dtype=np.float32) * np.float32(0.02))
    q = bf(g.standard_normal((Hg, 128), dtype=np.float32) / np.float32(11.3)); k = bf(g.standard_normal((Hg, 128), dtype=np.float32) / np.float32(11.3))
    v = bf(g.standard_normal((Hg, 128), dtype=np.float32))
    gl = (-np.log1p(np.exp(g.standard_normal(Hg))) * 0.1).astype(np.float32); beta = (1 / (1 + np.exp(-g.standard_normal(Hg)))).astype(np.float32)
    gdn_bytes = Hg * (2 * 128 * 128 * 4 + 3 * 128 * 2 + 128 * 2 + 8)
    orc.set_threads(all_threads)
    reps, dt = _timed(lambda: orc.gdn_core(q, k, v, gl, beta, S, Hg), seconds_per_op)
    ops["gdn_step"] = {"threads": all_threads, "value": round(reps * gdn_bytes / dt / 1e9, 3), "unit": "GB/s",
                       "us_per_step": round(dt / reps * 1e6, 1), "sample": f"{reps} x core recurrence, batch 1, 32 heads of 128x128, in {dt:.1f} s"}

    # paged decode attention (refAttn, prototypes/fa2_vllm.ts:114-139 for one query row): BASELINE configs[3], batch 1, L = 4096
    B, L, NH, NKV, HD = 1, 4096, 16, 2, 256
    kc, vc, bt, ctx = synth.paged_kv_random(g, B, L)
    qa = bf(g.standard_normal((B, NH, HD)).astype(np.float32))
    att_bytes = int(2 * NKV * int(ctx[0]) * HD * 2 + NH * HD * 2 * 2 + NH * 4)
    reps, dt = _timed(lambda: orc.attn_decode_paged(qa, kc, vc, bt, ctx, B, NH, NKV, HD, 16), seconds_per_op)
    ops["attn_decode"] = {"threads": all_threads, "value": round(reps * att_bytes / dt / 1e9, 3), "unit": "GB/s",
                          "us_per_call": round(dt / reps * 1e6, 1), "sample": f"{reps} x batch 1, context {int(ctx[0])} of 4096, 16 q / 2 KV heads, in {dt:.1f} s"}

    out = {"value": gemv["all_cores"]["value"], "unit": "GB/s", "cores": all_threads, "kind": "port",
           "sample": gemv["all_cores"]["sample"] + f" with the C oracle on {all_threads} OpenMP threads",
           "host": host, "ops": ops}
    if decode_inputs:
        out["decode_step"], parity = decode_parity(decode_inputs, all_threads)
        return out, parity
    return out, None


def decode_parity(decode_inputs, threads):
    """The checker decodes the same sequences on its own (timed: the CPU's tok/s for the full step) and its tokens are
    compared with the GPU's free run.  Every op but attention is equal bit for bit, so a token can differ only where the
    checker's top-1/top-2 margin is below the logit noise that one-ulp bf16 differences of the attention outputs leave;
    the step-by-step check that continues from the GPU's attention outputs (tests/test_gpu_model.py) demands equality."""
    from oracle import oracle as orc
    from oracle.model_ref import RefModel, free_run_report

    orc.set_threads(threads)
    D, W = decode_inputs["D"], decode_inputs["W"]
    timing, parity = {}, {}
    for key, (S, starts, pos0, toks, vals) in decode_inputs["runs"].items():
        ref = RefModel(D, W, S, batch=len(starts))
        steps = toks.shape[0]
        t0 = time.perf_counter()
        rt_, rv = ref.decode(starts, pos0, steps)
        dt = time.perf_counter() - t0
        rep = free_run_report(toks, vals, rt_, rv, np.array(ref.margins))
        rep["mode"] = "free run of both sides; strict step-by-step equality is tests/test_gpu_model.py"
        parity[key] = rep
        timing[key] = {"threads": threads, "value": round(steps * len(starts) / dt, 3), "unit": "tok/s",
                       "sample": f"{steps} steps x {len(starts)} sequence(s) of the synthetic model with the C oracle in {dt:.1f} s"}
    return timing, parity


def bench_decode(rt, synth, use_graph=True, steps_bs1=240, steps_bs32=48, fused=True):
    """tok/s of the full synthetic decode step at batch 1 and 32 (device-resident loop, HIP graph replay)."""
    from bunker_amd import model, runner, synth_model

    D = model.SYNTH
    W = synth_model.synth_weights(D, seed=2026)
    out = {}
    dev_w = None
    envs = []
    parity_runs = {}
    PARITY = {1: ([0], 32), 32: ([0, 13, 31], 16)}       # sequences and steps the checker decodes again on the CPU
    weight_bytes = sum(v.nbytes for k, v in W.items() if v.dtype == np.uint8)
    # the step as it ships (attention in double precision: the checker's bits) and, as a second figure, with the bf16
    # matrix-instruction attention (within 2e-2 per attention output; tokens then follow the checker only while the
    # top-1 / top-2 margin clears the noise)
    for B, steps, exact in ((1, steps_bs1, True), (32, steps_bs32, True), (1, steps_bs1, False), (32, steps_bs32, False)):
        if not exact:
            S = synth_model.device_state(synth_model.synth_state(D, batch=B, seed=7, share_kv_across_batch=True))
            g = model.buildModelGraph(D, B)
            env = runner.DecodeEnv(g, W, S, inplace_state=True, device_weights=dev_w)
            starts = [(9419 + 4099 * i) % D.VOCAB for i in range(B)]
            warm = 8 if B == 1 else 4
            loop = runner.DeviceLoop(g, env, B, starts, 4096, max_steps=warm + steps, use_graph=use_graph,
                                     partition=runner.fusedPartition(g) if fused else None, attn_exact=False)
            loop.step(warm)
            rt.cuSync()
            e0, e1 = rt.Event().record(), rt.Event()
            loop.step(steps)
            e1.record()
            rt.cuSync()
            ms = e0.elapsed_ms(e1) / steps
            out[f"bs{B}"]["with_bf16_mfma_attention"] = {"tok_per_s": round(B / (ms * 1e-3), 1), "ms_per_step": round(ms, 4)}
            loop.close()
            env.close()                    # its state; the weights belong to the first environment
            continue
        S_host = synth_model.synth_state(D, batch=B, seed=7, share_kv_across_batch=True)
        chk, nchk = PARITY[B]
        S_chk = {k: np.array(np.asarray(v)[chk], copy=True) for k, v in S_host.items()}
        S = synth_model.device_state(S_host)
        del S_host
        g = model.buildModelGraph(D, B)
        env = runner.DecodeEnv(g, W, S, inplace_state=True, device_weights=dev_w)
        envs.append(env)
        dev_w = dev_w or env.weight_ptrs()
        starts = [(9419 + 4099 * i) % D.VOCAB for i in range(B)]
        warm = 8 if B == 1 else 4          # warm + steps stays inside the KV capacity (4096 + 256 tokens)
        loop = runner.DeviceLoop(g, env, B, starts, 4096, max_steps=warm + steps, use_graph=use_graph,
                                 partition=runner.fusedPartition(g) if fused else None)
        loop.step(warm)
        rt.cuSync()
        e0, e1 = rt.Event(), rt.Event()
        t0 = time.perf_counter()
        e0.record()
        loop.step(steps)
        e1.record()
        rt.cuSync()
        wall = time.perf_counter() - t0
        ms = e0.elapsed_ms(e1) / steps
        toks, vals = loop.tokens()
        nchk = min(nchk, toks.shape[0])
        parity_runs[f"bs{B}"] = (S_chk, [starts[i] for i in chk], 4096, toks[:nchk][:, chk].copy(), vals[:nchk][:, chk].copy())
        # bytes one step must move: every Q4_K weight once, GDN state read+write, the KV prefix of the FA layers
        n_gdn = sum(1 for l in range(D.NL) if not D.is_full_attention(l))
        n_fa = D.NL - n_gdn
        state_bytes = B * n_gdn * (2 * D.LVH * D.LKD * D.LVD * 4) + B * n_fa * (2 * D.NKV * 4097 * D.HD * 2)
        floor_us = (weight_bytes + state_bytes) / 8e12 * 1e6
        out[f"bs{B}"] = {"tok_per_s": round(B / (ms * 1e-3), 1), "ms_per_step": round(ms, 4),
                         "wall_ms_per_step": round(wall * 1e3 / steps, 4), "steps": steps,
                         "launch": "hip graph replay" if use_graph else "eager", "ops_per_step": len(loop.launches), "kernel_launches_per_step": loop.graph_exec.node_count() if loop.graph_exec is not None else None, "partition": "fused" if fused else "node per kernel", "step_bytes": weight_bytes + state_bytes,
                         "hbm_floor_us": round(floor_us, 1), "frac_of_floor": round(floor_us / (ms * 1e3), 4),
                         "attention": "double precision (fa2 ops exact=1)",
                         "first_tokens": toks[:4, 0].tolist()}
    # prompt processing on the same model (sequence 0 of the batch-1 environment, from an empty state)
    from bunker_amd import prefill
    n_prompt, chunk = 2048, 1024
    pf = prefill.Prefill(D, envs[0], chunk=chunk)
    prompt = ((9419 + 7919 * np.arange(n_prompt, dtype=np.int64)) % D.VOCAB).astype(np.int32)
    pf.run(prompt, 0, 0)                   # loads the kernels of both chunks in flight
    rt.cuSync()
    t0 = time.perf_counter()
    tok, _ = pf.run(prompt, 0, 0)
    wall = time.perf_counter() - t0
    pf.close()
    out["prefill"] = {"prompt_tokens": n_prompt, "chunk": chunk, "chunks_in_flight": 2, "tok_per_s": round(n_prompt / wall, 1), "ms": round(wall * 1e3, 2),
                      "first_generated_token": tok, "attention": "double precision (the state T decode steps leave, bit for bit)"}
    pf = prefill.Prefill(D, envs[0], chunk=chunk, attn_exact=False)
    pf.run(prompt, 0, 0)
    rt.cuSync()
    t0 = time.perf_counter()
    pf.run(prompt, 0, 0)
    wall = time.perf_counter() - t0
    pf.close()
    out["prefill"]["with_bf16_mfma_attention"] = {"tok_per_s": round(n_prompt / wall, 1), "ms": round(wall * 1e3, 2),
                                                  "attention": "query tile x K/V tile on the bf16 matrix cores (fa2_prefill exact=0)"}
    # the reference's prefill forms on both ops that couple tokens: tiled bf16 attention and the chunked GDN recurrence
    pf = prefill.Prefill(D, envs[0], chunk=chunk, gdn_chunked=True, attn_exact=False)
    pf.run(prompt, 0, 0)
    rt.cuSync()
    t0 = time.perf_counter()
    tok_c, _ = pf.run(prompt, 0, 0)
    wall = time.perf_counter() - t0
    pf.close()
    out["prefill"]["with_tiled_attention_and_chunked_gdn"] = {"tok_per_s": round(n_prompt / wall, 1), "ms": round(wall * 1e3, 2),
                                                              "first_generated_token": tok_c,
                                                              "gdn": "chunks of 64 tokens on the f32 matrix instruction (gdn_prefill chunked=1)"}
    for env in envs:
        env.close()
    # the reference model's own dimensions (src/model.ts:14-18), random Q4_K weights, KV at 4096: batch 1 only
    from dataclasses import replace
    DR = replace(model.REFERENCE, MAX_LEN=4352)
    WR = synth_model.synth_weights(DR, seed=2027)
    SR = synth_model.device_state(synth_model.synth_state(DR, batch=1, seed=9))
    gR = model.buildModelGraph(DR, 1)
    envR = runner.DecodeEnv(gR, WR, SR, inplace_state=True)
    loopR = runner.DeviceLoop(gR, envR, 1, [9419], 4096, max_steps=8 + steps_bs1, use_graph=use_graph,
                              partition=runner.fusedPartition(gR) if fused else None)
    loopR.step(8)
    rt.cuSync()
    e0, e1 = rt.Event().record(), rt.Event()
    loopR.step(steps_bs1)
    e1.record()
    rt.cuSync()
    ms = e0.elapsed_ms(e1) / steps_bs1
    out["reference_dims"] = {"dims": "hidden 1024, FFN 3584, vocab 248320, 18 GDN + 6 attention layers (src/model.ts:14-18)",
                             "bs1": {"tok_per_s": round(1e3 / ms, 1), "ms_per_step": round(ms, 4), "steps": steps_bs1}}
    envR.close()
    return out, {"D": D, "W": W, "runs": parity_runs}


def bench_load(rt, synth):
    """Weights path: the Q4_K quantizer alone, and a bf16 safetensors file -> resident buffer (file read + PCIe)."""
    import os
    import tempfile
    from bunker_amd import loader

    rows, K = 32768, 2048
    g = synth.rng(99)
    w = synth.f32_to_bf16(g.standard_normal((rows, K), dtype=np.float32) * np.float32(0.02))
    d = rt.to_device(w)
    q = rt.cuAlloc(rows * (K // 256) * 144)
    rt.quantize_q4k(d, q, rows, K, rt.BF16)
    rt.cuSync()
    e0, e1 = rt.Event().record(), rt.Event()
    for _ in range(5):
        rt.quantize_q4k(d, q, rows, K, rt.BF16)
    e1.record(); rt.cuSync()
    ms = e0.elapsed_ms(e1) / 5
    rt.cuFree(d); rt.cuFree(q)
    out = {"quantize_q4k": {"rows": rows, "K": K, "ms": round(ms, 3), "gelem_per_s": round(rows * K / ms / 1e6, 2)}}
    tmp = tempfile.mkdtemp(prefix="bunker_bench_")
    path = os.path.join(tmp, "w.safetensors")
    loader.writeSafeTensors(path, {f"t{i}": ("BF16", w) for i in range(2)})
    size = os.path.getsize(path)
    loader.loadSafeTensors(path).free()
    t0 = time.perf_counter()
    f = loader.loadSafeTensors(path)
    dt = time.perf_counter() - t0
    f.free()
    os.remove(path); os.rmdir(tmp)
    out["load_safetensors"] = {"bytes": size, "ms": round(dt * 1e3, 1), "gb_per_s": round(size / dt / 1e9, 2),
                               "note": "page-cache-warm file -> pinned staging -> device, PCIe included"}
    return out


def bench_tokenizer():
    """gt_encode / gt_encode_mt (host C++, no GPU work) on this repository's own documents, with a vocabulary trained on
    them by the Hugging Face `tokenizers` library (whose encoder is timed beside ours); skipped where that library is absent."""
    try:
        from tokenizers import Regex, Tokenizer, models, pre_tokenizers, trainers
    except ImportError:
        return {"skipped": "the `tokenizers` package is not importable"}
    from bunker_amd import tokenizer
    root = os.path.dirname(os.path.abspath(__file__))
    text = "".join(open(os.path.join(root, f), encoding="utf-8").read() for f in ("bench.py", "bunker_amd/runner.py", "bunker_amd/loader.py"))
    qwen = r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+"
    tok = Tokenizer(models.BPE())
    tok.pre_tokenizer = pre_tokenizers.Sequence([pre_tokenizers.Split(Regex(qwen), behavior="isolated", invert=False),
                                                 pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=False)])
    tr = trainers.BpeTrainer(vocab_size=3000, special_tokens=["<|endoftext|>"], initial_alphabet=pre_tokenizers.ByteLevel.alphabet(),
                             show_progress=False)
    tok.train_from_iterator([text[i:i + 1500] for i in range(0, len(text), 1500)], tr)
    tmp = tempfile.mkdtemp(prefix="bk_tok_")
    path = os.path.join(tmp, "tokenizer.json")
    tok.save(path)
    t = tokenizer.Tokenizer(path)
    big = text * 16
    nbytes = len(big.encode("utf-8"))
    res = {"bytes": nbytes, "threads_mt": os.cpu_count()}
    ref_ids = None
    for name, fn in (("gt_encode", lambda: t.encode(big)), ("gt_encode_mt", lambda: t.encode(big, mt=True)),
                     ("hugging_face_tokenizers", lambda: np.asarray(tok.encode(big).ids))):
        fn()
        t0 = time.perf_counter()
        ids = fn()
        dt = time.perf_counter() - t0
        res[name] = {"MB_per_s": round(nbytes / dt / 1e6, 1), "ids": int(len(ids))}
        if name == "gt_encode":
            ref_ids = ids
        elif name == "hugging_face_tokenizers":
            res["gt_encode"]["equal_to_hugging_face"] = bool(len(ids) == len(ref_ids) and np.array_equal(np.asarray(ids), np.asarray(ref_ids)))
    t.close()
    os.remove(path); os.rmdir(tmp)
    return res


def _time_launches(rt, enqueue, use_graph):
    """Microseconds for everything `enqueue` launches, by HIP events on the library's stream."""
    e0, e1 = rt.Event(), rt.Event()
    if use_graph:
        with rt.Graph() as gr:
            enqueue()
        rt.cuSync()
        e0.record(); gr.launch(); e1.record()
    else:
        rt.cuSync()
        e0.record(); enqueue(); e1.record()
    rt.cuSync()
    return e0.elapsed_ms(e1) * 1e3


MFMA_INT8_PEAK_TOPS = 5000.0      # MI355X dense int8


def bench_gemm(rt, synth, use_graph=True, iters=60, batch=32):
    """The batched decode matmul (int8 MFMA, batch 32) at the decode shapes: weight GB/s and int8 TOP/s."""
    g = synth.rng(9)
    res = {}
    for name, N, K in SHAPES:
        h = synth.q4k_random(g, N, K)
        n = max(2, int(-(-ROTATION_BYTES // h.nbytes)))
        first = rt.to_device(h)
        ws = [first]
        for _ in range(n - 1):
            p = rt.cuAlloc(h.nbytes); rt.cuDtoD(p, first, h.nbytes); ws.append(p)
        dx = rt.to_device(g.standard_normal((batch, K)).astype(np.float32))
        xq = rt.cuAlloc(batch * (K // 32) * 36)
        rt.quantize_q8_1(dx, xq, K, batch, rt.F32)
        y = rt.cuAlloc(batch * N * 4)
        for i in range(10):
            rt.gemm_q4k_q8_1(ws[i % n], xq, y, N, K, batch)
        us = _time_launches(rt, lambda: [rt.gemm_q4k_q8_1(ws[i % n], xq, y, N, K, batch) for i in range(iters)], use_graph) / iters
        nbytes = gemv_bytes(N, K, batch)
        tops = 2.0 * N * K * batch / us / 1e6
        res[name] = {"N": N, "K": K, "batch": batch, "us": round(us, 3), "bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1),
                     "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "int8_TOPs": round(tops, 1),
                     "frac_mfma_int8_peak": round(tops / MFMA_INT8_PEAK_TOPS, 5)}
        for p in ws + [dx, xq, y]:
            rt.cuFree(p)
    return res


def bench_kernels(rt, synth, use_graph=True, iters=50):
    """Gated-DeltaNet step (configs[2]) and paged decode attention (configs[3]) in algorithmic GB/s."""
    g = synth.rng(5)
    res = {}
    bf = synth.f32_to_bf16
    for B in (1, 8):
        Hg = 32
        ROT = max(2, 600 // (B * Hg * 131072 // (1 << 20) + 1))      # rotate states through > 512 MiB
        ROT = min(ROT, 140)
        S = (g.standard_normal((B, Hg, 128, 128), dtype=np.float32) * np.float32(0.02))
        dS = [rt.to_device(S) for _ in range(ROT)]
        q = rt.to_device(bf(g.standard_normal((B, Hg, 128), dtype=np.float32) / np.float32(11.3)))
        k = rt.to_device(bf(g.standard_normal((B, Hg, 128), dtype=np.float32) / np.float32(11.3)))
        v = rt.to_device(bf(g.standard_normal((B, Hg, 128), dtype=np.float32)))
        gl = rt.to_device((-np.log1p(np.exp(g.standard_normal((B, Hg)))) * 0.1).astype(np.float32))
        beta = rt.to_device((1 / (1 + np.exp(-g.standard_normal((B, Hg))))).astype(np.float32))
        dout = rt.cuAlloc(B * Hg * 128 * 2)
        for i in range(5):
            rt.gdn_core(q, k, v, gl, beta, dS[i % ROT], dout, dS[i % ROT], Hg, B)
        def run_gdn():
            for i in range(iters):
                rt.gdn_core(q, k, v, gl, beta, dS[i % ROT], dout, dS[i % ROT], Hg, B)

        us = _time_launches(rt, run_gdn, use_graph) / iters
        nbytes = B * Hg * (2 * 128 * 128 * 4 + 3 * 128 * 2 + 128 * 2 + 8)
        res[f"gdn_step_b{B}"] = {"us": round(us, 3), "bytes": nbytes, "GBps": round(nbytes / us / 1e3, 1),
                                 "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
        for p in dS + [q, k, v, gl, beta, dout]:
            rt.cuFree(p)
    for B, L in ((1, 4096), (8, 4096), (1, 32768), (8, 32768)):
        NH, NKV, HD = 16, 2, 256
        ppseq = L // 16
        ctx = g.integers(L // 2, L + 1, B).astype(np.int32)
        bt = g.permutation(B * ppseq).astype(np.int32).reshape(B, ppseq)
        page = bf(g.standard_normal((64, NKV, 16, HD), dtype=np.float32))
        reps = (B * ppseq + 63) // 64
        cache = np.tile(page, (reps, 1, 1, 1))[: B * ppseq]
        ROT = max(2, min(8, int(600e6 // (2 * cache.nbytes)) + 1))
        kcs = [rt.to_device(cache) for _ in range(ROT)]
        vcs = [rt.to_device(cache) for _ in range(ROT)]
        dq = rt.to_device(bf(g.standard_normal((B, NH, HD), dtype=np.float32)))
        dbt, dctx = rt.to_device(bt), rt.to_device(ctx)
        dout, dlse = rt.cuAlloc(B * NH * HD * 2), rt.cuAlloc(B * NH * 4)
        nbytes = int(sum(2 * NKV * int(c) * HD * 2 for c in ctx) + B * NH * HD * 2 * 2 + B * NH * 4)
        # the matrix-instruction form (bf16 products, 2e-2) and the double-precision form (the checker's bits; the
        # default of the decode step's attention op)
        for key, plan, fn in (("attn_decode", rt.attn_plan, rt.attn_decode), ("attn_decode_exact", rt.attn_plan_exact, rt.attn_decode_exact)):
            splits, ws = plan(B, NKV, L)
            dws = rt.cuAlloc(ws) if ws else 0

            def run(i):
                fn(dq, kcs[i % ROT], vcs[i % ROT], dbt, ppseq, dctx, L, dout, dlse, B, NH, NKV, HD, 16, splits, dws, ws)

            for i in range(3):
                run(i)
            us = _time_launches(rt, lambda: [run(i) for i in range(iters)], use_graph) / iters
            res[f"{key}_b{B}_L{L}"] = {"us": round(us, 3), "bytes": nbytes, "splits": splits,
                                       "GBps": round(nbytes / us / 1e3, 1),
                                       "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
            if dws:
                rt.cuFree(dws)
        dws = 0
        for p in kcs + vcs + [dq, dbt, dctx, dout, dlse] + ([dws] if dws else []):
            rt.cuFree(p)
    res.update(bench_prefill_ops(rt, synth))
    return res


def bench_fused_ops(rt, synth, use_graph=True, iters=48, batches=(1, 32)):
    """The fused ops the decode step is made of, each on its own (one stream, weights and state rotated through 24
    copies like the 24 layers of the step): microseconds per launch and algorithmic GB/s.  The same launches a decode
    step makes, without the device loop, the prompt pass or a second stream around them."""
    g = synth.rng(21)
    bf = synth.f32_to_bf16
    H, I, Hg, NH, NKV, HD, MAXL, POS = 2048, 6144, 16, 16, 2, 256, 4352, 4096
    ROT = 24
    res = {}

    def q4k(N, K):
        h = synth.q4k_random(g, N, K)
        first = rt.to_device(h)
        out = [first]
        for _ in range(ROT - 1):
            p = rt.cuAlloc(h.nbytes); rt.cuDtoD(p, first, h.nbytes); out.append(p)
        return out, h.nbytes

    def time_op(key, spec, args_of, nbytes, owned):
        k = rt.compileAndLoad(spec)
        def launch(i):
            rc = rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], args_of(i))
            if rc != 0:
                raise rt.BunkerError(f"{spec}: {rt.last_error()}")
        for i in range(3):
            launch(i)
        us = _time_launches(rt, lambda: [launch(i) for i in range(iters)], use_graph) / iters
        res[key] = {"spec": spec, "us": round(us, 3), "bytes": int(nbytes), "GBps": round(nbytes / us / 1e3, 1),
                    "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
        rt.unloadKernel(k)
        for p in owned:
            rt.cuFree(p)

    for B in batches:
        bp = f" batch={B}" if B != 1 else ""
        q8 = B >= 8
        x = rt.to_device(bf(g.standard_normal((B, H), dtype=np.float32)))
        nw = rt.to_device(bf((g.standard_normal(H) * 0.1).astype(np.float32)))
        resid = rt.to_device(bf(g.standard_normal((B, H), dtype=np.float32)))
        # GDN layer.  Batch < 8 (slab form): rmsnorm + qkv (+ conv1d), z, a, b | recurrence in four column slabs per head,
        # raw outputs | gated norm + out_proj + residual add.  Batched: rmsnorm + qkv, z, a, b | conv1d + recurrence |
        # out_proj + add reading the recurrence's Q8_1 copy.
        slab = not q8
        C = 3 * Hg * 128
        (Wqkv, b0), (Wz, b1), (Wa, b2), (Wb, b3) = q4k(C, H), q4k(Hg * 128, H), q4k(Hg, H), q4k(Hg, H)
        oq, oz, oa, ob = rt.cuAlloc(B * C * 2), rt.cuAlloc(B * Hg * 128 * 2), rt.cuAlloc(B * Hg * 4), rt.cuAlloc(B * Hg * 4)
        st = [rt.to_device(bf(g.standard_normal((B, 3, C), dtype=np.float32))) for _ in range(ROT)]
        cw = rt.to_device(bf((g.standard_normal((C, 4)) * 0.5).astype(np.float32)))
        conv_bytes = B * C * 2 * 6 + C * 8         # three state rows in and out, the taps
        if slab:
            time_op(f"gdn_projections_conv_b{B}", f"gemv_fused K={H} pro=2 G=4 N0={C} epi0=3 N1={Hg * 128} epi1=1 N2={Hg} epi2=0 N3={Hg} epi3=0" + bp,
                    lambda i: [x, nw, Wqkv[i % ROT], st[i % ROT], cw, oq, st[i % ROT], Wz[i % ROT], oz, Wa[i % ROT], oa, Wb[i % ROT], ob],
                    b0 + b1 + b2 + b3 + B * H * 2 + B * (4 * Hg * 128) * 2 + conv_bytes, Wqkv + Wz + Wa + Wb + [oa, ob])
        else:
            time_op(f"gdn_projections_b{B}", f"gemv_fused K={H} pro=2 G=4 N0={C} epi0=1 N1={Hg * 128} epi1=1 N2={Hg} epi2=0 N3={Hg} epi3=0" + bp,
                    lambda i: [x, nw, Wqkv[i % ROT], oq, Wz[i % ROT], oz, Wa[i % ROT], oa, Wb[i % ROT], ob],
                    b0 + b1 + b2 + b3 + B * H * 2 + B * (4 * Hg * 128) * 2, Wqkv + Wz + Wa + Wb + [oa, ob])
        A_log = rt.to_device(g.uniform(-2, 1, Hg).astype(np.float32)); dtb = rt.to_device(bf(g.standard_normal(Hg).astype(np.float32)))
        ap = rt.to_device(g.standard_normal((B, Hg)).astype(np.float32)); bpp = rt.to_device(g.standard_normal((B, Hg)).astype(np.float32))
        gw = rt.to_device((1 + 0.1 * g.standard_normal(128)).astype(np.float32))
        S0 = (g.standard_normal((B, Hg, 128, 128), dtype=np.float32) * np.float32(0.02))
        dS = [rt.to_device(S0) for _ in range(ROT)]
        rt.cuHtoD(oq, bf(g.standard_normal((B, C), dtype=np.float32))); rt.cuHtoD(oz, bf(g.standard_normal((B, Hg * 128), dtype=np.float32)))
        gout = rt.cuAlloc(B * Hg * 128 * 2); gq8 = rt.cuAlloc(B * Hg * 4 * 36); graw = rt.cuAlloc(B * (Hg * 128 * 8 + Hg * 32))
        state_bytes = B * Hg * (2 * 128 * 128 * 4)
        if slab:
            time_op(f"gdn_slabs_b{B}", f"gdn_slabs LVH={Hg} LKD=128 LVD=128" + bp,
                    lambda i: [oq, oz, A_log, dtb, ap, bpp, dS[i % ROT], graw, dS[i % ROT]],
                    state_bytes + B * (C * 2 + Hg * 128 * 2 + Hg * 128 * 8 + Hg * 32), dS + st + [cw, A_log, dtb, ap, bpp, oq, oz])
        else:
            time_op(f"gdn_conv_b{B}", f"gdn_conv LVH={Hg} LKD=128 LVD=128" + bp + " q8out=1",
                    lambda i: [oq, st[i % ROT], cw, oz, A_log, dtb, ap, bpp, gw, dS[i % ROT], gout, st[i % ROT], dS[i % ROT], gq8],
                    state_bytes + B * C * 2 + conv_bytes + B * Hg * 128 * 4, st + dS + [cw, A_log, dtb, ap, bpp, oq, oz])
        Wo, bo = q4k(H, Hg * 128)
        hout = rt.cuAlloc(B * H * 2)
        if slab:
            time_op(f"out_proj_gated_norm_add_b{B}", f"gemv_fused K={Hg * 128} pro=3 G=1 N0={H} epi0=2" + bp,
                    lambda i: [graw, gw, Wo[i % ROT], resid, hout], bo + B * (Hg * 128 * 8 + 2 * H * 2), Wo + [gout, gq8, graw, gw])
        else:
            time_op(f"out_proj_add_b{B}", f"gemv_fused K={Hg * 128} pro=0 G=1 N0={H} epi0=2" + bp,
                    lambda i: [gq8, Wo[i % ROT], resid, hout], bo + B * (Hg * 128 * 2 + 2 * H * 2), Wo + [gout, gq8, graw, gw])
        # MLP: rmsnorm + gate, up + SwiGLU, then down + residual add
        (Wg, bg), (Wu, bu), (Wd, bd) = q4k(I, H), q4k(I, H), q4k(H, I)
        act = rt.cuAlloc(B * I * 2); aq8 = rt.cuAlloc(B * (I // 32) * 36)
        time_op(f"gate_up_swiglu_b{B}", f"gemv_fused K={H} pro=2 G=2 swiglu=1 N0={I} N1={I}" + bp + (" q8out=1" if q8 else ""),
                lambda i: [x, nw, Wg[i % ROT], Wu[i % ROT], act] + ([aq8] if q8 else []), bg + bu + B * (H + I) * 2, Wg + Wu)
        time_op(f"down_add_b{B}", f"gemv_fused K={I} pro={0 if q8 else 1} G=1 N0={H} epi0=2" + bp,
                lambda i: [aq8 if q8 else act, Wd[i % ROT], resid, hout], bd + B * (I * 2 + 2 * H * 2), Wd + [act, aq8])
        # attention layer: rmsnorm + q|gate, k, v; norms + rope + append + attention over 4096 cached tokens; o_proj + add
        (Wq, bq), (Wk, bk), (Wv, bv), (Wop, bop) = q4k(2 * NH * HD, H), q4k(NKV * HD, H), q4k(NKV * HD, H), q4k(H, NH * HD)
        qg, kk, vv = rt.cuAlloc(B * 2 * NH * HD * 2), rt.cuAlloc(B * NKV * HD * 2), rt.cuAlloc(B * NKV * HD * 2)
        time_op(f"attn_projections_b{B}", f"gemv_fused K={H} pro=2 G=3 N0={2 * NH * HD} epi0=1 N1={NKV * HD} epi1=1 N2={NKV * HD} epi2=1" + bp,
                lambda i: [x, nw, Wq[i % ROT], qg, Wk[i % ROT], kk, Wv[i % ROT], vv], bq + bk + bv + B * H * 2 + B * (2 * NH + 2 * NKV) * HD * 2,
                Wq + Wk + Wv)
        for buf, n in ((qg, B * 2 * NH * HD), (kk, B * NKV * HD), (vv, B * NKV * HD)):
            rt.cuHtoD(buf, bf(g.standard_normal(n, dtype=np.float32)))
        page = bf(g.standard_normal((64, NKV, 16, HD), dtype=np.float32))
        cache = np.tile(page, ((B * (MAXL // 16) + 63) // 64, 1, 1, 1))[: B * (MAXL // 16)]
        NR = 6 if B == 1 else 3
        kcs = [rt.to_device(cache) for _ in range(NR)]; vcs = [rt.to_device(cache) for _ in range(NR)]
        cos_t = rt.to_device(g.uniform(-1, 1, (MAXL, 32)).astype(np.float32)); sin_t = rt.to_device(g.uniform(-1, 1, (MAXL, 32)).astype(np.float32))
        qw = rt.to_device(bf((g.standard_normal(HD) * 0.1).astype(np.float32))); kw = rt.to_device(bf((g.standard_normal(HD) * 0.1).astype(np.float32)))
        dpos = rt.to_device(np.full(B, POS, np.int32))
        aout = rt.cuAlloc(B * NH * HD * 2); attq8 = rt.cuAlloc(B * (NH * HD // 32) * 36)
        time_op(f"fa2_fused_b{B}_ctx{POS}", f"fa2_fused HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} ROT_HALF=32 pos_dev=1" + bp + (" q8out=1" if q8 else ""),
                lambda i: [qg, kk, vv, qw, kw, cos_t, sin_t, dpos, kcs[i % NR], vcs[i % NR], aout] + ([attq8] if q8 else []),
                B * (2 * NKV * (POS + 1) * HD * 2 + (2 * NH + 2 * NKV + NH) * HD * 2), kcs + vcs + [cos_t, sin_t, qw, kw, dpos, qg, kk, vv])
        time_op(f"o_proj_add_b{B}", f"gemv_fused K={NH * HD} pro={0 if q8 else 1} G=1 N0={H} epi0=2" + bp,
                lambda i: [attq8 if q8 else aout, Wop[i % ROT], resid, hout], bop + B * (NH * HD * 2 + 2 * H * 2), Wop + [aout, attq8, hout])
        for p in (x, nw, resid):
            rt.cuFree(p)
    return res


MFMA_BF16_PEAK_TFLOPS = 2500.0     # MI355X dense bf16
MFMA_F32_PEAK_TFLOPS = 157.3       # MI355X f32 matrix


def bench_prefill_ops(rt, synth, iters=5):
    """The two prompt ops that couple the tokens of a sequence, each in its forms: causal attention of 1024 prompt tokens
    behind 15360 cached ones (fa2_prefill: norms, rotation and cache append included) and the Gated-DeltaNet recurrence
    over 1024 tokens of 16 heads (gdn_prefill: gates, norms and the output norm included)."""
    g = synth.rng(15)
    bf = synth.f32_to_bf16
    res = {}

    def timed(spec, args):
        h = rt.compileAndLoad(spec)
        for _ in range(2):
            rt.cuLaunch(h, [1, 1, 1], [128, 1, 1], args)
        us = _time_launches(rt, lambda: [rt.cuLaunch(h, [1, 1, 1], [128, 1, 1], args) for _ in range(iters)], False) / iters
        rt.unloadKernel(h)
        return us

    NH, NKV, HD, HALF, MAXL, T, pos0 = 16, 2, 256, 32, 16384, 1024, 15360
    pages = MAXL // 16
    page = bf(g.standard_normal((64, NKV, 16, HD), dtype=np.float32))
    cache = np.tile(page, (pages // 64, 1, 1, 1))
    host = (bf(g.standard_normal((T, NH, 2, HD), dtype=np.float32)), bf(g.standard_normal((T, NKV, HD), dtype=np.float32)),
            bf(g.standard_normal((T, NKV, HD), dtype=np.float32)), bf((g.standard_normal(HD) * 0.1).astype(np.float32)),
            bf((g.standard_normal(HD) * 0.1).astype(np.float32)), g.uniform(-1, 1, (MAXL, HALF)).astype(np.float32),
            g.uniform(-1, 1, (MAXL, HALF)).astype(np.float32), (pos0 + np.arange(T)).astype(np.int32), np.arange(pages, dtype=np.int32))
    ptrs = [rt.to_device(a) for a in host] + [rt.to_device(cache), rt.to_device(cache), rt.cuAlloc(T * NH * HD * 2)]
    spec = f"fa2_prefill HD={HD} NH={NH} NKV={NKV} MAX_LEN={MAXL} ROT_HALF={HALF} T={T}"
    flop = float(sum(pos0 + t + 1 for t in range(T))) * NH * 4 * HD            # 2 products x 2 flop per (row, token, dim)
    row = {"prompt_tokens": T, "cached_tokens": pos0, "flop": flop}
    for key, flags in (("tiled_bf16_mfma", " exact=0"), ("decode_kernel_per_token_pair", " exact=0 tiled=0"), ("double_precision", "")):
        us = timed(spec + flags, ptrs)
        row[key] = {"us": round(us, 1), "TFLOPs": round(flop / us / 1e6, 1)}
    row["tiled_bf16_mfma"]["frac_bf16_mfma_peak"] = round(row["tiled_bf16_mfma"]["TFLOPs"] / MFMA_BF16_PEAK_TFLOPS, 4)
    res["fa2_prefill_T1024_behind_15360"] = row
    for p in ptrs:
        rt.cuFree(p)

    Hg, T = 16, 1024
    C = 3 * Hg * 128
    host = (bf(g.standard_normal((T, C), dtype=np.float32)), bf(g.standard_normal((T, Hg * 128), dtype=np.float32)),
            g.uniform(-2, 1, Hg).astype(np.float32), bf(g.standard_normal(Hg).astype(np.float32)),
            (g.standard_normal((T, Hg)) * 2).astype(np.float32), g.standard_normal((T, Hg)).astype(np.float32),
            (1 + 0.1 * g.standard_normal(128)).astype(np.float32), (g.standard_normal((Hg, 128, 128)) * 0.02).astype(np.float32))
    ptrs = [rt.to_device(a) for a in host]
    args = ptrs + [rt.cuAlloc(T * Hg * 128 * 2), rt.cuAlloc(host[7].nbytes)]
    # chunked form: per chunk of 64 tokens and head, products of 64x64x128 (K K^T, Q K^T), 2 x 64x64x128 (W, Uv),
    # 2 x 64x128x128 (W S, K^T U), 64x128x128 (Q S) and 64x64x128 (M U): 11 M multiply-adds
    flop_chunked = 2.0 * 11 * 64 * 64 * 128 * (T // 64) * Hg
    row = {"tokens": T, "heads": Hg,
           "scan": {"us": round(timed(f"gdn_prefill LVH={Hg} T={T}", args), 1)},
           "chunked_f32_mfma": {"us": round(timed(f"gdn_prefill LVH={Hg} T={T} chunked=1", args), 1)}}
    row["chunked_f32_mfma"]["TFLOPs"] = round(flop_chunked / row["chunked_f32_mfma"]["us"] / 1e6, 2)
    row["chunked_f32_mfma"]["frac_f32_mfma_peak"] = round(row["chunked_f32_mfma"]["TFLOPs"] / MFMA_F32_PEAK_TFLOPS, 4)
    res["gdn_prefill_T1024_H16"] = row
    for p in args:
        rt.cuFree(p)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # 2000 timed steps after 500 warm-up steps by default; a fixed, untimed clock warm-up (PREWARM_S) runs in front of
    # them whatever --steps says, because the clocks of an idle GPU take a few thousand launches to settle (without it
    # the same kernels measured 8 % slower in a 20- or 200-step run)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sections", default="gemv,decode,kernels,gemm,fused,load,tok",
                    help="comma list of gemv (headline, always on), decode (with prefill), kernels, gemm, fused (the decode step's "
                         "fused ops one by one), calib, load (weights path), tok (tokenizer, host only)")
    ap.add_argument("--mode", choices=["graph", "stream"], default="graph",
                    help="GEMV section. graph: the K launches of a shape replayed from one HIP graph (the device's own launch "
                         "rate); stream: K individual launches per shape queued from the host (used under rocprofv3)")
    ap.add_argument("--unfused", action="store_true", help="decode section: one kernel per graph node (the reference's partition)")
    ap.add_argument("--no-graph", action="store_true",
                    help="decode and kernels sections launch eagerly instead of replaying HIP graphs "
                         "(rocprofv3 cannot trace graph launches on this ROCm)")
    args = ap.parse_args()
    # under rocprofv3 the decode and kernels sections launch eagerly: its tracer faults inside hipGraphLaunch on this ROCm
    profiled = "rocprof" in os.environ.get("LD_PRELOAD", "") or any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ)
    if profiled:
        args.no_graph = True
        args.mode = "stream"
        print("bench.py: profiler attached, every section launches from the host instead of replaying HIP graphs", file=sys.stderr)
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no collectives, no sharding).", file=sys.stderr)
        sys.exit(2)

    from bunker_amd import runtime as rt
    from bunker_amd import synth

    rt.cu(0)
    info = rt.device_info()
    g = synth.rng(2026)

    # per shape: as many device copies of the matrix as it takes to span ROTATION_BYTES (launches are grouped by shape,
    # so each shape needs its own > 256 MiB working set: 85 copies of qkv and down, 43 of gate_up, 4 of lm_head)
    copies = {}        # copies[shape] = [device pointers]
    for name, N, K in SHAPES:
        h = synth.q4k_random(g, N, K)
        n = max(2, int(-(-ROTATION_BYTES // h.nbytes)))
        first = rt.to_device(h)
        copies[name] = [first]
        for _ in range(n - 1):
            p = rt.cuAlloc(h.nbytes)
            rt.cuDtoD(p, first, h.nbytes)
            copies[name].append(p)
        del h
    xq, y = {}, {}
    for name, N, K in SHAPES:
        x = g.standard_normal(K).astype(np.float32)
        dx = rt.to_device(x)
        xq[name] = rt.cuAlloc(K // 32 * 36)
        rt.quantize_q8_1(dx, xq[name], K, 1, rt.F32)
        y[name] = rt.cuAlloc(N * 4)
    rt.cuSync()

    def launch(name, N, K, i):
        rt.gemv_q4k_q8_1(copies[name][i % len(copies[name])], xq[name], y[name], N, K)

    # each shape: one HIP graph of K launches (graph mode), W warm-up launches of that shape directly before its timed
    # K launches, an event on either side.  The timed region of the workload is the sum of the four: exactly K steps.
    graphs = {}
    if args.mode == "graph":
        for name, N, K in SHAPES:
            with rt.Graph() as gr:
                for i in range(args.steps):
                    launch(name, N, K, i)
            graphs[name] = gr
        rt.cuSync()

    def run_region(name, N, K, n):
        e0, e1 = rt.Event(), rt.Event()
        for w in range(args.warmup):
            launch(name, N, K, w)
        if args.mode == "graph":
            # one untimed replay directly in front of the timed one: the timed replay is then queued while the device
            # is still busy, so its K launches are measured at the device's own rate even when K is small (a lone
            # 20-launch replay also pays the host's submission latency, +0.5 us per launch)
            graphs[name].launch()
        e0.record()
        if args.mode == "graph":
            graphs[name].launch()
        else:
            for i in range(n):
                launch(name, N, K, i)
        e1.record()
        rt.cuSync()
        return e0.elapsed_ms(e1)

    # duration of the shortest possible launch in the same mode (16-byte read by one workgroup): the floor under every
    # kernel here, and the reason the three small shapes cannot come near the HBM roofline
    sink = rt.cuAlloc(256)
    n_floor = 500
    for _ in range(20):
        rt.memread(sink, 16, sink + 128)
    rt.cuSync()
    if args.mode == "graph":
        with rt.Graph() as gfl:
            for _ in range(n_floor):
                rt.memread(sink, 16, sink + 128)
        rt.cuSync()

    def measure_floor():
        f0, f1 = rt.Event(), rt.Event()
        f0.record()
        if args.mode == "graph":
            gfl.launch()
        else:
            for _ in range(n_floor):
                rt.memread(sink, 16, sink + 128)
        f1.record()
        rt.cuSync()
        return f0.elapsed_ms(f1) * 1e3 / n_floor

    # Untimed clock warm-up of fixed length, so that a short run (--steps 20) is measured at the clocks a long one
    # settles at: the clocks of an idle GPU take a few thousand launches to come up.  The same GEMV launches as the timed
    # region, all four shapes in turn, for PREWARM_S seconds of wall time; --steps / --warmup keep their meaning.
    launch_floor_cold_us = measure_floor()
    t_pw = time.perf_counter()
    while time.perf_counter() - t_pw < PREWARM_S:
        for name, N, K in SHAPES:
            for i in range(100 if N < 100000 else 25):
                launch(name, N, K, i)
        rt.cuSync()
    prewarm_ms = (time.perf_counter() - t_pw) * 1e3
    launch_floor_us = measure_floor()
    rt.cuFree(sink)

    t0 = time.perf_counter()
    region_ms = {name: run_region(name, N, K, args.steps) for name, N, K in SHAPES}
    wall = time.perf_counter() - t0

    per_shape = {}
    total_ms = sum(region_ms.values())
    for si, (name, N, K) in enumerate(SHAPES):
        ms = region_ms[name] / args.steps
        b = gemv_bytes(N, K)
        body_us = max(ms * 1e3 - launch_floor_us, 1e-3)      # what the kernel adds to the shortest possible launch
        per_shape[name] = {"N": N, "K": K, "us_per_launch": round(ms * 1e3, 3), "bytes": b,
                           "GBps": round(b / (ms * 1e-3) / 1e9, 1),
                           "frac_hbm_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                           "us_minus_launch_floor": round(body_us, 3),
                           "GBps_minus_launch_floor": round(b / body_us / 1e3, 1),
                           "frac_hbm_peak_minus_launch_floor": round(b / body_us / 1e3 / HBM_PEAK_GBS, 4)}
    step_bytes = sum(gemv_bytes(N, K) for _, N, K in SHAPES)
    ms_per_step = total_ms / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # dominant kernel: the instantiation with the largest share of the step.  Rows of 2048 run as
    # gemv_q4k_q8_1_lds_kernel<1,0,RPI> with RPI = 2 rows per wave step up to 16384 rows and 4 above (lm_head);
    # rows of 6144 as <3,0,2>.
    def kernel_of(N, K):
        return f"gemv_q4k_q8_1_lds_kernel<{K // 2048},0,{4 if (K == 2048 and N > 16384) else 2}>"
    by_kernel = {}
    for n, N, K in SHAPES:
        by_kernel.setdefault(kernel_of(N, K), []).append(n)
    dom_kernel, dom = max(by_kernel.items(), key=lambda kv: sum(per_shape[n]["us_per_launch"] for n in kv[1]))
    dom_bytes = sum(per_shape[n]["bytes"] for n in dom) / len(dom)
    dom_us = sum(per_shape[n]["us_per_launch"] for n in dom) / len(dom)
    achieved = dom_bytes / (dom_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "kernel": dom_kernel, "shapes": dom, "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "avg_launch_us": round(dom_us, 3), "bytes_per_launch": int(dom_bytes),
                "traffic": measured_traffic(dom_kernel, "+".join(dom))}

    out = {
        "metric": "Q4_K GEMV HBM GB/s (% of peak); synthetic Qwen3.5 decode tok/s at bs=1/32",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u4 x int8 -> int32 dots, f64 fold, f32 out", "data": "synthetic",
        "config": {"workload": "Q4_K x Q8_1 GEMV, batch 1, decode shapes qkv/gate_up/down/lm_head "
                               "(BASELINE configs[1]); one step = one launch of each shape",
                   "weight_rotation_MB_per_shape": {n: round(len(c) * NN * KK * 144 // 256 / 1e6) for (n, NN, KK), c in
                                                    zip(SHAPES, copies.values())},
                   "launch_mode": args.mode, "device": info["name"], "cus": info["cus"]},
        "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "launch_floor_us": round(launch_floor_us, 3),
        "launch_floor_before_prewarm_us": round(launch_floor_cold_us, 3),
        "prewarm_ms": round(prewarm_ms, 1),
        "wall_ms_per_step_incl_warmup": round(wall * 1e3 / args.steps, 5),
        "per_shape": per_shape,
        "roofline": roofline,
    }
    for c in copies.values():
        for p in c:
            rt.cuFree(p)
    sections = set(args.sections.split(","))
    if "calib" in sections:
        # a plain copy of known size, for scaling the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run
        nb = 175030272
        a, b = rt.cuAlloc(nb), rt.cuAlloc(nb)
        rt.cuMemset(a, 1, nb)
        for _ in range(10):
            rt.memcopy(a, b, nb)
        rt.cuSync()
        rt.cuFree(a); rt.cuFree(b)
        out["calib"] = {"kernel": "memcopy_kernel", "bytes_read": nb, "bytes_written": nb, "launches": 10}
    decode_inputs = None
    if "decode" in sections:
        out["decode"], decode_inputs = bench_decode(rt, synth, use_graph=not args.no_graph, fused=not args.unfused)
        if args.no_cpu_baseline:
            decode_inputs = None
    if "kernels" in sections:
        out["kernels"] = bench_kernels(rt, synth, use_graph=not args.no_graph)
    if "gemm" in sections:
        out["gemm_bs32"] = bench_gemm(rt, synth, use_graph=not args.no_graph)
    if "fused" in sections:
        out["fused_ops"] = bench_fused_ops(rt, synth, use_graph=not args.no_graph)
    if "load" in sections:
        out["weights_path"] = bench_load(rt, synth)
    if "tok" in sections:
        out["tokenizer"] = bench_tokenizer()
    if not args.no_cpu_baseline:
        out["cpu_baseline"], parity = cpu_baseline(decode_inputs)
        for key, rep in (parity or {}).items():
            out["decode"][key]["argmax_parity"] = rep
    print(json.dumps(out))


if __name__ == "__main__":
    main()
