"""Full decode step on the GPU against the CPU restatement.

Every op of the step shares its arithmetic rules with the checker and is equal to it bit for bit,
attention included (its double-precision form is the default of the fa2_* ops).  Two checks:

* strict: step by step, the checker recomputes the step from the same state and tokens; every
  attention output of the GPU, all logits, the winning logit, the argmax token id and the
  recurrent state must be EQUAL;
* free-running: both sides decode on their own for the whole run; every token id and every
  winning logit must be equal, whatever the top-1/top-2 margin (reported) is.

TINY has the model's structure at small dims; SYNTH is the benchmark's synthetic Qwen3.5-style
model (BASELINE configs[4]) with KV prefilled to 4096."""
import numpy as np
import pytest

from bunker_amd import model, runner, synth_model
from bunker_amd import runtime as rt
from bunker_amd.model import SYNTH, TINY

pytestmark = pytest.mark.gpu


def _fa_layers(D):
    return [l for l in range(D.NL) if D.is_full_attention(l)]


def _strict_decode(D, W, S, starts, pos0, steps, use_graph, check=None, fused=False, device_weights=None):
    """GPU DeviceLoop one token at a time against the checker continued from the GPU's attention outputs.

    check: the sequences of the batch the checker recomputes (all by default; sequences are independent)."""
    from oracle.model_ref import RefModel
    B = len(starts)
    check = list(range(B)) if check is None else list(check)
    g = model.buildModelGraph(D, B)
    env = runner.DecodeEnv(g, W, synth_model.device_state(S), inplace_state=True, device_weights=device_weights)
    loop = runner.DeviceLoop(g, env, B, starts, pos0, max_steps=steps, use_graph=use_graph,
                             partition=runner.fusedPartition(g) if fused else None)
    fa_nodes = [n for n in g.nodes if n.op == "fa2_attn"]
    logits_name = next(n for n in g.nodes if n.op == "argmax").inputs[0].tensorName
    ref = RefModel(D, W, {k: np.asarray(v)[check] for k, v in S.items()}, batch=len(check))
    toks = np.asarray(starts, np.int32)[check]; pos = np.full(len(check), pos0, np.int32)
    for step in range(steps):
        loop.step(1)
        rt.cuSync()
        inj = {l: rt.from_device(env.resolve(n.outputs[0].tensorName), (B, D.NH * D.HD), np.uint16)[check]
               for l, n in zip(_fa_layers(D), fa_nodes)}
        glogits = rt.from_device(env.resolve(logits_name), (B, D.VOCAB), np.float32)[check]
        idx, val, rlogits = ref.step(toks, pos, attn_override=inj)
        gt, gv = loop.tokens()
        assert np.array_equal(glogits.view(np.uint32), rlogits.view(np.uint32)), \
            f"step {step}: {int((glogits != rlogits).sum())} logits differ, worst {np.abs(glogits - rlogits).max():.3e}"
        assert np.array_equal(gt[step][check], idx) and np.array_equal(gv[step][check].view(np.uint32), val.view(np.uint32)), \
            (step, gt[step], idx)
        toks, pos = idx, pos + 1
    print("strict: tokens", loop.tokens()[0].T.tolist(), "max attention |gpu-ref| %.3g" % max(ref.attn_err), flush=True)
    assert max(ref.attn_err) == 0.0          # the double-precision attention returns the checker's bits
    # recurrent state after the last token
    for l in range(D.NL):
        p = f"model.layers.{l}"
        if not D.is_full_attention(l):
            Sg = env.read_state(f"{p}.s_state", (B, D.LVH, 128, 128), np.float32)[check]
            assert np.array_equal(Sg.view(np.uint32), ref.S[f"{p}.s_state"].view(np.uint32)), p
            cg = env.read_state(f"{p}.conv_state", (B, 3, D.QKVD), np.uint16)[check]
            assert np.array_equal(cg, ref.S[f"{p}.conv_state"]), p
        else:
            kg = env.read_state(f"{p}.kv_k", (B,) + ref.S[f"{p}.kv_k"].shape[1:], np.uint16)[check]
            assert np.array_equal(kg, ref.S[f"{p}.kv_k"]), p
            vg = env.read_state(f"{p}.kv_v", (B, D.MAX_LEN // 16, D.NKV, D.HD, 16), np.uint16)[check].swapaxes(-1, -2)
            assert np.array_equal(vg, ref.S[f"{p}.kv_v"]), p
    env.close()
    return loop.tokens()


def _free_running(D, W, S, starts, pos0, steps, got_tokens, got_vals):
    """Both sides decode on their own: every op returns the checker's bits, so tokens and winning logits are equal for the
    whole run however small the top-1/top-2 margin gets (it is printed: random weights give near-ties)."""
    from oracle.model_ref import RefModel, free_run_report
    ref = RefModel(D, W, S, batch=len(starts))
    rt_, rv = ref.decode(starts, pos0, steps)
    margins = np.array(ref.margins)
    rep = free_run_report(got_tokens, got_vals, rt_, rv, margins)
    print("free-running:", rep, flush=True)
    assert np.array_equal(got_tokens, rt_), rep
    assert np.array_equal(got_vals.view(np.uint32), rv.view(np.uint32)), rep
    return rep


def test_tiny_model_reference_loop(orc):
    """The reference's host loop (scalars per launch, double-buffered state) on the tiny model."""
    D = TINY
    W = synth_model.synth_weights(D, seed=11)
    S = synth_model.synth_state(D, batch=1, seed=12)
    steps, pos0 = 6, 40
    g = model.buildModelGraph(D, 1)
    env = runner.DecodeEnv(g, W, synth_model.device_state(S))
    compiled = runner.compileStep(g, runner.choosePartition(g))
    out = runner.runGraphDecode(compiled, env.resolve, 77, steps, lambda t, v, s: env.rotateState(), startPos=pos0)
    toks = np.array(out["tokens"], np.int32)[:, None]; vals = np.array(out["logits"], np.float32)[:, None]
    st, sv = _strict_decode(D, W, S, [77], pos0, steps, use_graph=False)
    # the host loop and the device-resident loop run the same kernels: same tokens, same logits, bit for bit
    assert np.array_equal(toks, st) and np.array_equal(vals.view(np.uint32), sv.view(np.uint32))
    _free_running(D, W, S, [77], pos0, steps, toks, vals)
    env.close()


@pytest.mark.parametrize("use_graph,fused", [(False, False), (True, False), (False, True), (True, True)])
def test_tiny_model_device_loop_batch3(orc, use_graph, fused):
    D = TINY
    W = synth_model.synth_weights(D, seed=11)
    S = synth_model.synth_state(D, batch=3, seed=13)
    toks, vals = _strict_decode(D, W, S, [77, 5, 900], 40, 20, use_graph, fused=fused)      # 19 replays of the recorded step
    _free_running(D, W, S, [77, 5, 900], 40, 20, toks, vals)


@pytest.mark.parametrize("fused", [False, True])
def test_synthetic_qwen35_decode_step_bs1(orc, fused):
    """BASELINE configs[4], batch 1: 24 layers (3 GDN : 1 FA), hidden 2048, FFN 6144, vocab 151936, KV at 4096.
    fused: the partition with the fused kernels (138 launches per token instead of 425); same bits."""
    D = SYNTH
    print("generating weights", flush=True)
    W = synth_model.synth_weights(D, seed=2026)
    S = synth_model.synth_state(D, batch=1, seed=7)
    # 32 tokens on the benchmark's partition (the reference's own bar is 31 matching tokens, prototypes/decode.ts:933);
    # the node-per-kernel partition runs the same kernels one by one and keeps a short run
    steps, pos0, tok0 = (32 if fused else 6), 4096, 9419     # start token of the reference's benches (bench_graph_decode.ts:77)
    toks, vals = _strict_decode(D, W, S, [tok0], pos0, steps, use_graph=True, fused=fused)
    _free_running(D, W, S, [tok0], pos0, steps, toks, vals)


def test_tiny_model_batch32_mfma_path(orc):
    """Batch 32 sends every matmul through the int8 MFMA kernel; results stay equal to the checker's."""
    D = TINY
    W = synth_model.synth_weights(D, seed=11)
    S = synth_model.synth_state(D, batch=32, seed=14)
    starts = [(37 * i + 5) % D.VOCAB for i in range(32)]
    toks, vals = _strict_decode(D, W, S, starts, 40, 16, use_graph=True)
    tf, vf = _strict_decode(D, W, S, starts, 40, 16, use_graph=True, fused=True)
    assert np.array_equal(tf, toks) and np.array_equal(vf.view(np.uint32), vals.view(np.uint32))
    # a sequence decodes to the same tokens alone (GEMV path) as inside the batch (MFMA path)
    S1 = {k: np.asarray(v)[7:8] for k, v in S.items()}
    t1, v1 = _strict_decode(D, W, S1, [starts[7]], 40, 16, use_graph=False)
    assert np.array_equal(t1[:, 0], toks[:, 7]) and np.array_equal(v1[:, 0].view(np.uint32), vals[:, 7].view(np.uint32))


def test_synthetic_qwen35_decode_step_bs32(orc):
    """BASELINE configs[4], batch 32: 32 different start tokens and states, int8 MFMA matmuls; three of
    the sequences are recomputed by the checker."""
    D = SYNTH
    W = synth_model.synth_weights(D, seed=2026)
    S = synth_model.synth_state(D, batch=32, seed=8, share_kv_across_batch=True)
    starts = [(9419 + 4099 * i) % D.VOCAB for i in range(32)]
    check = [0, 13, 31]
    toks, vals = _strict_decode(D, W, S, starts, 4096, 16, use_graph=True, check=check, fused=True)
    _free_running(D, W, {k: np.asarray(v)[check] for k, v in S.items()}, [starts[i] for i in check], 4096, 16,
                  toks[:, check], vals[:, check])


@pytest.mark.parametrize("batch", [1, 9])
def test_reference_dims_decode(orc, batch):
    """The dimensions of src/model.ts:14-18 (hidden 1024, FFN 3584, 8 query heads) with 4 layers and a short vocabulary:
    K = 1024 and 3584 are outside the fused GEMV's fast path, so the same op specs run their composed form
    (RMSNorm -> Q8_1 kernel, generic-K GEMV at batch 1, MFMA matmul at batch 9) and must give the same bits."""
    from dataclasses import replace
    D = replace(model.REFERENCE, NL=4, VOCAB=4096, MAX_LEN=64)
    print(f"reference dims, batch {batch}", flush=True)
    W = synth_model.synth_weights(D, seed=41)
    S = synth_model.synth_state(D, batch=batch, seed=42)
    starts = [(113 * i + 9) % D.VOCAB for i in range(batch)]
    toks, vals = _strict_decode(D, W, S, starts, 30, 3, use_graph=True, fused=True, check=[0, batch - 1] if batch > 1 else None)
    assert toks.shape == (3, batch)


@pytest.mark.parametrize("seed", [100, 104, 106, 109])
def test_free_running_decode_equals_the_checker_over_seeds(orc, seed):
    """No injection, no step-by-step resynchronisation: 4 sequences decode 23 tokens on the GPU (fused partition, replayed
    graph) and on the CPU from the same weights and state; tokens and winning logits must be equal although the top-1 /
    top-2 margins of random weights fall below 1e-3 (seeds 106, 109)."""
    from oracle.model_ref import RefModel
    D, B, steps = TINY, 4, 23
    pos0 = 5 + seed % 30
    W = synth_model.synth_weights(D, seed=seed)
    S = synth_model.synth_state(D, batch=B, seed=seed + 1)
    g = model.buildModelGraph(D, B)
    env = runner.DecodeEnv(g, W, synth_model.device_state(S), inplace_state=True)
    starts = [(17 + 911 * i + seed) % D.VOCAB for i in range(B)]
    loop = runner.DeviceLoop(g, env, B, starts, pos0, max_steps=steps, use_graph=True, partition=runner.fusedPartition(g))
    loop.step(steps)
    toks, vals = loop.tokens()
    ref = RefModel(D, W, S, batch=B)
    rtok, rv = ref.decode(starts, pos0, steps)
    print(f"seed {seed}: min margin {np.min(ref.margins):.5f}", flush=True)
    assert np.array_equal(toks, rtok) and np.array_equal(vals.view(np.uint32), rv.view(np.uint32))
    # the replayed graph holds at least one kernel per op and not many more (an op is one to three launches)
    assert len(loop.launches) <= loop.graph_exec.node_count() <= 3 * len(loop.launches)
    loop.close(); env.close()


def test_token_feedback_forms_agree(orc):
    """argmax_feed (argmax's second stage + token feedback + the next embedding in one launch) against argmax, advance and the
    step's own embed launch: same tokens, same logits."""
    D, B, steps = TINY, 3, 9
    W = synth_model.synth_weights(D, seed=41)
    S = synth_model.synth_state(D, batch=B, seed=42)
    g = model.buildModelGraph(D, B)
    res = []
    for feed in (True, False):
        env = runner.DecodeEnv(g, W, synth_model.device_state(S), inplace_state=True)
        loop = runner.DeviceLoop(g, env, B, [3, 700, 41], 20, max_steps=steps, use_graph=True, partition=runner.fusedPartition(g), feed=feed)
        assert (len(loop.first_only) == 1) == feed
        loop.step(steps)
        res.append(loop.tokens())
        loop.close(); env.close()
    assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1].view(np.uint32), res[1][1].view(np.uint32))
