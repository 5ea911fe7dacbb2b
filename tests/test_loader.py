"""Checkpoint formats and the weight quantizer's checker, on the CPU.

The 144-byte super-block quantizer restates the published ggml fit; ggml itself is absent, so equality with
ggml's bytes is unpinned and the checks here are the ones the mathematics fixes: the fp16 rounding against
numpy's, the fit against the plain min/max grid it starts from, exactly affine data, constant blocks, and the
half-step reconstruction bound of the stored block."""
import numpy as np
import pytest

from bunker_amd import loader, synth
from oracle import oracle as orc

bf = synth.f32_to_bf16


def test_f32_to_half_rne_matches_numpy_and_round_trips():
    hs = np.arange(65536, dtype=np.uint16)
    vals = hs.view(np.float16).astype(np.float32)
    for h, v in zip(hs[::7], vals[::7]):
        if not np.isnan(v):
            assert orc.f32_to_half_rne(v) == h
    g = synth.rng(5)
    x = (g.standard_normal(4000) * np.exp(g.uniform(-20, 12, 4000))).astype(np.float32)
    # exact midpoints between neighbouring halves: ties go to the even mantissa
    lo = np.arange(0x0001, 0x7bff, 37, dtype=np.uint16)
    mid = (lo.view(np.float16).astype(np.float64) + (lo + 1).astype(np.uint16).view(np.float16).astype(np.float64)) / 2
    x = np.concatenate([x, mid.astype(np.float32), -mid.astype(np.float32), np.float32([0, -0.0, 65504, 65519.99, 65520, 1e9, 6e-8, 2.9e-8, 3.1e-8])])
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    got = np.array([orc.f32_to_half_rne(v) for v in x], np.uint16)
    assert np.array_equal(got, ref)


def _werr(x, w, scale, mn, L):
    return float(np.sum(w.astype(np.float64) * (scale * L.astype(np.float64) + mn - x.astype(np.float64)) ** 2))


def test_fit_is_never_worse_than_the_min_max_grid():
    g = synth.rng(11)
    for trial in range(200):
        x = (g.standard_normal(32) * np.exp(g.uniform(-6, 2))).astype(np.float32)
        if trial % 3 == 0:
            x += np.float32(g.uniform(-1, 1))
        w = (np.sqrt(np.mean(x.astype(np.float64) ** 2)) + np.abs(x)).astype(np.float32)
        scale, the_min, L = orc.qkx2_fit32(x, w)
        assert L.max() <= 15
        mn = min(float(x.min()), 0.0); mx = float(x.max())
        if mx == mn:
            continue
        s0 = (mx - mn) / 15
        L0 = np.clip(np.rint((x.astype(np.float64) - mn) / s0), 0, 15)
        assert _werr(x, w, scale, -the_min, L) <= _werr(x, w, s0, mn, L0) * (1 + 1e-4) + 1e-12
        assert the_min >= 0


def test_fit_recovers_affine_data():
    g = synth.rng(12)
    for _ in range(50):
        L = g.integers(0, 16, 32); L[:2] = [0, 15]
        a, b = float(np.exp(g.uniform(-5, 0))), -float(np.exp(g.uniform(-5, 0)))
        x = (a * L + b).astype(np.float32)
        w = (np.sqrt(np.mean(x.astype(np.float64) ** 2)) + np.abs(x)).astype(np.float32)
        scale, the_min, Lq = orc.qkx2_fit32(x, w)
        assert np.array_equal(Lq, L)
        assert abs(scale - a) <= 1e-4 * a and abs(the_min + b) <= 1e-4 * abs(b) + 1e-6 * a


def test_constant_and_zero_blocks():
    z = orc.quantize_q4k(np.zeros(256, np.float32))
    assert not z.any()
    c = orc.quantize_q4k(np.full(256, -0.5, np.float32))
    assert np.allclose(orc.q4k_dequant(c), -0.5, rtol=2e-3)         # d = 0, everything rides on dmin * 63
    assert c[16:].max() == 0
    p = orc.quantize_q4k(np.full(256, 0.25, np.float32))
    assert np.allclose(orc.q4k_dequant(p), 0.25, rtol=2e-3)


@pytest.mark.parametrize("sigma", [0.02, 1.0, 2e-4])
def test_stored_block_reconstructs_within_half_a_step(sigma):
    g = synth.rng(13)
    x = (g.standard_normal((8, 1024)) * sigma).astype(np.float32)
    q = orc.quantize_q4k(x).reshape(-1, 144)
    y = orc.q4k_dequant(q).reshape(-1, 8, 32)
    xs = x.reshape(-1, 8, 32).astype(np.float64)
    for b in range(q.shape[0]):
        d = orc.half_to_float(int(q[b, 0]) | int(q[b, 1]) << 8); dmin = orc.half_to_float(int(q[b, 2]) | int(q[b, 3]) << 8)
        sc, m = np.zeros(8, np.uint8), np.zeros(8, np.uint8)
        import ctypes as C
        orc.lib().orc_q4k_unpack_scales(q[b, 4:16].ctypes.data_as(C.c_void_p), sc.ctypes.data_as(C.c_void_p), m.ctypes.data_as(C.c_void_p))
        assert sc.max() == 63 or d == 0
        for j in range(8):
            step, off = d * float(sc[j]), dmin * float(m[j])
            if step == 0:
                continue
            t = (xs[b, j] + off) / step
            inside = (t >= 0) & (t <= 15)
            assert np.all(np.abs(y[b, j][inside] - xs[b, j][inside]) <= 0.5 * step * (1 + 1e-4) + 1e-12)
    rel = np.sqrt(np.mean((y.reshape(x.shape) - x) ** 2) / np.mean(x.astype(np.float64) ** 2))
    assert rel < 0.09, rel          # 4-bit blocks with fitted scales on Gaussian data


def test_safetensors_round_trip(tmp_path):
    g = synth.rng(21)
    tensors = {"a.weight": ("BF16", bf(g.standard_normal((3, 5)).astype(np.float32))),
               "b": ("F32", g.standard_normal(7).astype(np.float32)),
               "c": ("I64", np.arange(4, dtype=np.int64))}
    p = str(tmp_path / "m.safetensors")
    loader.writeSafeTensors(p, tensors, {"format": "pt"})
    header, meta, start, size = loader.readSafeTensorsHeader(p)
    assert meta == {"format": "pt"} and set(header) == set(tensors) and start % 16 == 0
    raw = open(p, "rb").read()
    for name, (dt, arr) in tensors.items():
        b, e = header[name]["data_offsets"]
        assert header[name]["dtype"] == dt and header[name]["shape"] == list(arr.shape)
        assert b % 16 == 0 or arr.nbytes % 16           # tensors of whole 16-byte pieces come first, aligned
        assert raw[start + b:start + e] == arr.tobytes()
    spans = sorted(h["data_offsets"] for h in header.values())        # no gaps: the format allows none
    assert spans[0][0] == 0 and all(a[1] == b[0] for a, b in zip(spans, spans[1:])) and spans[-1][1] == size - start
    with open(p, "r+b") as f:                       # a header that claims more bytes than the file has
        f.truncate(size - 8)
    with pytest.raises(ValueError):
        loader.readSafeTensorsHeader(p)


def test_safetensors_against_the_safetensors_package(tmp_path):
    """Both directions against the published implementation of the format (the `safetensors` package): a file this
    writer makes is read back by the package, and a file the package writes (tensors packed back to back, sorted by
    dtype and name, its own header padding) is parsed by this reader to the same bytes."""
    st = pytest.importorskip("safetensors")
    import safetensors.numpy as stnp
    g = synth.rng(23)
    f32 = g.standard_normal((5, 3)).astype(np.float32)
    f16 = g.standard_normal(11).astype(np.float16)
    i32 = g.integers(-9, 9, (2, 2, 2)).astype(np.int32)
    one = np.array(3.5, np.float32)                          # a scalar: shape []
    # ours -> theirs (bf16 is not a numpy dtype: the package reads it through its header only, checked as raw bytes)
    bfa = bf(g.standard_normal((4, 6)).astype(np.float32))
    p1 = str(tmp_path / "ours.safetensors")
    loader.writeSafeTensors(p1, {"x.f32": ("F32", f32), "x.f16": ("F16", f16.view(np.uint16)), "x.i32": ("I32", i32),
                                 "x.bf16": ("BF16", bfa), "x.one": ("F32", one)}, {"format": "pt", "n": 3})
    back = stnp.load_file(p1) if not _has_bf16(p1) else None
    with st.safe_open(p1, framework="numpy") as f:
        assert set(f.keys()) == {"x.f32", "x.f16", "x.i32", "x.bf16", "x.one"} and f.metadata() == {"format": "pt", "n": "3"}
        assert np.array_equal(f.get_tensor("x.f32"), f32) and np.array_equal(f.get_tensor("x.f16"), f16)
        assert np.array_equal(f.get_tensor("x.i32"), i32) and f.get_tensor("x.one").shape == () and f.get_tensor("x.one") == 3.5
        sl = f.get_slice("x.bf16")
        assert sl.get_shape() == [4, 6] and sl.get_dtype() == "BF16"
    assert back is None
    # theirs -> ours
    p2 = str(tmp_path / "theirs.safetensors")
    stnp.save_file({"b.f32": f32, "a.f16": f16, "c.i32": i32, "d.one": one, "e.i64": np.arange(5, dtype=np.int64)}, p2,
                   metadata={"who": "package"})
    header, meta, start, size = loader.readSafeTensorsHeader(p2)
    assert meta == {"who": "package"} and set(header) == {"b.f32", "a.f16", "c.i32", "d.one", "e.i64"}
    raw = open(p2, "rb").read()
    want = {"b.f32": ("F32", f32), "a.f16": ("F16", f16), "c.i32": ("I32", i32), "d.one": ("F32", one),
            "e.i64": ("I64", np.arange(5, dtype=np.int64))}
    for name, (dt, arr) in want.items():
        b, e = header[name]["data_offsets"]
        assert header[name]["dtype"] == dt and header[name]["shape"] == list(arr.shape)
        assert raw[start + b:start + e] == arr.tobytes(), name
    assert max(h["data_offsets"][1] for h in header.values()) == size - start       # the data section ends with the file


def _has_bf16(path):
    return any(v.get("dtype") == "BF16" for k, v in loader.readSafeTensorsHeader(path)[0].items())


def test_gguf_round_trip(tmp_path):
    g = synth.rng(22)
    q = synth.q4k_centered(g, 4, 512, 0.02)
    tensors = {"w": (loader.GGML_Q4_K, [4, 512], q), "n": (loader.GGML_BF16, [9], bf(g.standard_normal(9).astype(np.float32))),
               "f": (loader.GGML_F32, [2, 3], g.standard_normal((2, 3)).astype(np.float32))}
    p = str(tmp_path / "m.gguf")
    loader.writeGGUF(p, tensors, {"qwen35.hidden": 2048, "general.name": "t", "x.f": 1.5, "x.b": True})
    meta, infos, start = loader.readGGUF(p)
    assert meta["general.architecture"] == "qwen35" and meta["qwen35.hidden"] == 2048 and meta["general.name"] == "t"
    assert meta["x.f"] == 1.5 and meta["x.b"] is True and start % 32 == 0
    raw = open(p, "rb").read()
    assert raw[:4] == b"GGUF"
    by = {i.name: i for i in infos}
    for name, (t, shape, arr) in tensors.items():
        i = by[name]
        assert i.shape == shape and i.ggml_type == t and i.offset % 32 == 0
        assert raw[start + i.offset:start + i.offset + i.nbytes] == np.ascontiguousarray(arr).tobytes()
    with pytest.raises(ValueError):
        loader.writeGGUF(p, {"bad": (loader.GGML_Q4_K, [4, 100], np.zeros(10, np.uint8))})


def test_safe_key_follows_the_checkpoint_naming():
    W = {"model.language_model.embed_tokens.weight": 1, "model.language_model.norm.weight": 2,
         "model.language_model.layers.3.mlp.up_proj.weight": 3, "rope_cos": 4}
    assert loader.safeKey("embed.weight", W) == "model.language_model.embed_tokens.weight"
    assert loader.safeKey("lm_head.weight", W) == "model.language_model.embed_tokens.weight"      # tied
    assert loader.safeKey("final.norm.weight", W) == "model.language_model.norm.weight"
    assert loader.safeKey("model.layers.3.mlp.up_proj.weight", W) == "model.language_model.layers.3.mlp.up_proj.weight"
    assert loader.safeKey("model.layers.4.mlp.up_proj.weight", W) is None
    assert loader.safeKey("rope_cos", W) == "rope_cos"
    W["lm_head.weight"] = 5
    assert loader.safeKey("lm_head.weight", W) == "lm_head.weight"
