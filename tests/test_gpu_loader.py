"""Weight path on the GPU: the Q4_K quantizer against the CPU checker (equal bytes), and a checkpoint file
-> resident weights -> decode, against the checker run on the same quantized weights."""
import numpy as np
import pytest

from bunker_amd import loader, model, synth, synth_model
from bunker_amd import runtime as rt
from bunker_amd.model import TINY, L

pytestmark = pytest.mark.gpu

bf = synth.f32_to_bf16
f32 = synth.bf16_to_f32


def _quantize_dev(w, dtype):
    d = rt.to_device(w)
    rows, K = w.shape
    out = rt.cuAlloc(rows * (K // 256) * 144)
    rt.cuMemset(out, 0xCD, rows * (K // 256) * 144)
    rt.quantize_q4k(d, out, rows, K, dtype)
    rt.cuSync()
    got = rt.from_device(out, (rows * (K // 256) * 144,), np.uint8)
    rt.cuFree(d); rt.cuFree(out)
    return got


def _special_rows(g, K):
    """Rows that reach the quantizer's branches: zeros, constants of either sign, one outlier, all positive,
    tiny and huge magnitudes (fp16 subnormal / large d), exactly affine data, ties at half steps."""
    rows = [np.zeros(K), np.full(K, -0.5), np.full(K, 0.25), np.abs(g.standard_normal(K)) * 0.1,
            g.standard_normal(K) * 1e-6, g.standard_normal(K) * 3e3, -np.abs(g.standard_normal(K)),
            (g.integers(0, 16, K) * 0.125 - 0.5), (g.integers(0, 31, K) * 0.0625 - 1.0)]
    o = g.standard_normal(K) * 0.01; o[::97] = 3.0
    rows.append(o)
    z = g.standard_normal(K) * 0.02; z[256:512] = 0.0; z[512:544] = 0.7
    rows.append(z)
    return np.stack(rows).astype(np.float32)


@pytest.mark.parametrize("rows,K,sigma", [(3, 256, 0.02), (64, 2048, 0.02), (5, 6144, 1.0), (37, 1024, 2e-4)])
def test_quantize_q4k_bf16_equals_checker(orc, rows, K, sigma):
    print(f"quantize_q4k bf16 rows={rows} K={K} sigma={sigma}", flush=True)
    g = synth.rng(4000 + rows + K)
    w = bf(np.concatenate([(g.standard_normal((rows, K)) * sigma).astype(np.float32), _special_rows(g, K)]))
    got = _quantize_dev(w, rt.BF16)
    ref = orc.quantize_q4k(f32(w))
    bad = np.flatnonzero(got != ref)
    assert bad.size == 0, f"{bad.size} bytes differ, first in block {bad[0] // 144} at byte {bad[0] % 144}"


@pytest.mark.parametrize("rows,K", [(2, 512), (33, 2048)])
def test_quantize_q4k_f32_equals_checker(orc, rows, K):
    print(f"quantize_q4k f32 rows={rows} K={K}", flush=True)
    g = synth.rng(4100 + rows)
    w = np.concatenate([(g.standard_normal((rows, K)) * np.exp(g.uniform(-8, 2, (rows, 1)))).astype(np.float32), _special_rows(g, K)])
    got = _quantize_dev(w, rt.F32)
    ref = orc.quantize_q4k(w)
    bad = np.flatnonzero(got != ref)
    assert bad.size == 0, f"{bad.size} bytes differ, first in block {bad[0] // 144} at byte {bad[0] % 144}"


def test_quantize_q4k_rejects_bad_shapes():
    d = rt.to_device(np.zeros(512, np.float32))
    with pytest.raises(rt.BunkerError):
        rt.quantize_q4k(d, d, 1, 300, rt.F32)
    with pytest.raises(rt.BunkerError):
        rt.quantize_q4k(d + 4, d, 1, 256, rt.F32)
    rt.cuFree(d)


def _checkpoint(D, seed):
    """bf16 tensors under the checkpoint's names (model.language_model.layers.N...), tied embedding."""
    g = synth.rng(seed)
    T = {}

    def lin(name, N, K):
        T[name] = ("BF16", bf((g.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)))

    def norm(name, n):
        T[name] = ("BF16", bf((g.standard_normal(n) * 0.02).astype(np.float32)))

    T["model.language_model.embed_tokens.weight"] = ("BF16", bf(g.standard_normal((D.VOCAB, D.H)).astype(np.float32)))
    for l in range(D.NL):
        p = f"model.language_model.layers.{l}"
        norm(f"{p}.input_layernorm.weight", D.H); norm(f"{p}.post_attention_layernorm.weight", D.H)
        if not D.is_full_attention(l):
            la = f"{p}.linear_attn"
            lin(f"{la}.in_proj_qkv.weight", D.QKVD, D.H); lin(f"{la}.in_proj_z.weight", D.ZD, D.H)
            lin(f"{la}.in_proj_a.weight", D.LVH, D.H); lin(f"{la}.in_proj_b.weight", D.LVH, D.H)
            lin(f"{la}.out_proj.weight", D.H, D.ZD)
            T[f"{la}.conv1d.weight"] = ("BF16", bf((g.standard_normal((D.QKVD, 4)) * 0.5).astype(np.float32)))
            T[f"{la}.A_log"] = ("F32", (g.standard_normal(D.LVH) * 0.5).astype(np.float32))
            T[f"{la}.dt_bias"] = ("BF16", bf(g.standard_normal(D.LVH).astype(np.float32)))
            T[f"{la}.norm.weight"] = ("BF16", bf((1.0 + 0.02 * g.standard_normal(D.LVD)).astype(np.float32)))   # graph wants f32
        else:
            sa = f"{p}.self_attn"
            lin(f"{sa}.q_proj.weight", D.QGATE, D.H); lin(f"{sa}.k_proj.weight", D.KV_DIM, D.H)
            lin(f"{sa}.v_proj.weight", D.KV_DIM, D.H); lin(f"{sa}.o_proj.weight", D.H, D.NH * D.HD)
            norm(f"{sa}.q_norm.weight", D.HD); norm(f"{sa}.k_norm.weight", D.HD)
        lin(f"{p}.mlp.gate_proj.weight", D.INTER, D.H); lin(f"{p}.mlp.up_proj.weight", D.INTER, D.H)
        lin(f"{p}.mlp.down_proj.weight", D.H, D.INTER)
    norm("model.language_model.norm.weight", D.H)
    return T


def _expected_weights(orc, D, T, graph):
    """What the loader must leave on the device, computed with the checker's quantizer."""
    W = {}
    for name, t in graph.tensors.items():
        if t.role != "weight":
            continue
        if name in ("rope_cos", "rope_sin"):
            continue
        key = loader.safeKey(name, T)
        dt, arr = T[key]
        if t.type.dtype == "q4_k":
            W[name] = orc.quantize_q4k(f32(arr) if dt == "BF16" else arr)
        elif t.type.dtype == "f32" and dt == "BF16":
            W[name] = f32(arr)
        else:
            W[name] = arr
    W["rope_cos"], W["rope_sin"] = synth_model.rope_tables(D)
    return W


@pytest.mark.parametrize("align", [16, 2])
def test_checkpoint_to_decode(orc, tmp_path, align):
    """safetensors (tensors packed back to back when align=2) -> loadQwen35 -> the bytes the checker's quantizer
    gives -> a decode that equals the checker's on those weights; then the GGUF copy of the resident model."""
    print(f"checkpoint -> decode, align={align}", flush=True)
    from test_gpu_model import _strict_decode
    D = TINY
    T = _checkpoint(D, 77)
    if align == 2:
        T = {"pad": ("BF16", np.zeros(1, np.uint16)), **T}
    path = str(tmp_path / "tiny.safetensors")
    loader.writeSafeTensors(path, T, {"format": "pt"}, align=align)
    g = model.buildModelGraph(D, 1)
    m = loader.loadQwen35(path, D, g)
    W = _expected_weights(orc, D, T, g)
    for name, ref in W.items():
        got = m.host_weight(g, name)
        assert np.array_equal(got, np.ascontiguousarray(ref).view(np.uint8).ravel()), name
    assert m.quantized_bytes == sum(v.nbytes for k, v in W.items() if g.tensors[k].type.dtype == "q4_k")

    S = synth_model.synth_state(D, 1, seed=3)
    toks, _ = _strict_decode(D, W, S, [5], 20, 4, use_graph=True, fused=True, device_weights=m.weights)
    assert toks.shape[0] == 4

    gpath = str(tmp_path / "tiny.gguf")
    loader.saveGGUF(m, gpath, g)
    m2 = loader.loadQwen35(gpath, D, g)
    for name in W:
        assert np.array_equal(m2.host_weight(g, name), m.host_weight(g, name)), name
    assert m2.quantized_bytes == 0
    meta, infos, _ = loader.readGGUF(gpath)
    assert meta["qwen35.hidden"] == D.H and {i.name for i in infos} == set(W) - {"rope_cos", "rope_sin"}
    m2.free(); m.free()


def test_load_reports_missing_and_misshapen_tensors(tmp_path):
    D = TINY
    T = _checkpoint(D, 78)
    g = model.buildModelGraph(D, 1)
    T2 = dict(T); del T2["model.language_model.layers.0.mlp.up_proj.weight"]
    p = str(tmp_path / "a.safetensors"); loader.writeSafeTensors(p, T2)
    with pytest.raises(KeyError, match="up_proj"):
        loader.loadQwen35(p, D, g)
    T3 = dict(T); dt, a = T3["model.language_model.layers.1.mlp.down_proj.weight"]
    T3["model.language_model.layers.1.mlp.down_proj.weight"] = (dt, a[:, :256].copy())
    p = str(tmp_path / "b.safetensors"); loader.writeSafeTensors(p, T3)
    with pytest.raises(ValueError, match="down_proj"):
        loader.loadQwen35(p, D, g)
