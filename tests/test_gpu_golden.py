"""The kernels against the committed known-answer fixtures of tests/golden/, through the C ABI."""
import numpy as np
import pytest

from bunker_amd import runtime as rt
from test_golden import argmax_input, bits_f32, gold

pytestmark = pytest.mark.gpu


def test_q8_1_blocks_gpu():
    for b in gold("q8_1_blocks.json")["blocks"]:
        dx = rt.to_device(bits_f32(b["x_f32_bits"])); dq = rt.cuAlloc(36)
        rt.quantize_q8_1(dx, dq, 32, 1, rt.F32)
        got = rt.from_device(dq, (36,), np.uint8)
        assert got[:32].view(np.int8).tolist() == b["q"]
        assert int(got[32:34].view(np.uint16)[0]) == b["d_half_bits"] and int(got[34:36].view(np.uint16)[0]) == b["s_half_bits"]
        rt.cuFree(dx); rt.cuFree(dq)


def test_legacy_dequant_gpu():
    blocks = gold("legacy_dequant.json")["blocks"]
    raw = np.array([b["block_bytes"] for b in blocks], np.uint8)
    d_in, d_out = rt.to_device(raw), rt.cuAlloc(len(blocks) * 32)
    rt.dequant_legacy_i8(d_in, d_out, len(blocks))
    got = rt.from_device(d_out, (len(blocks), 32), np.int8)
    assert got.tolist() == [b["int8"] for b in blocks]
    rt.cuFree(d_in); rt.cuFree(d_out)


def test_q4k_block_gpu():
    g = gold("q4k_block.json")
    d_in = rt.to_device(np.array(g["block_bytes"], np.uint8))
    d_n, d_w = rt.cuAlloc(256), rt.cuAlloc(256 * 4)
    rt.q4k_nibbles(d_in, d_n, 1); rt.q4k_dequant_f32(d_in, d_w, 1)
    assert rt.from_device(d_n, (256,), np.uint8).tolist() == g["nibbles"]
    w = rt.from_device(d_w, (256,), np.float32); ref = bits_f32(g["w_f32_bits_exact_rounded_once"])
    assert np.all(np.abs(w.astype(np.float64) - ref) <= np.spacing(np.abs(ref)).astype(np.float64) * 2)
    for p in (d_in, d_n, d_w):
        rt.cuFree(p)


def test_gemv_q4k_q8_1_gpu():
    g = gold("gemv_q4k_q8_1.json")
    N, K = g["N"], g["K"]
    dW = rt.to_device(np.array(g["W_bytes"], np.uint8))
    dx = rt.to_device(bits_f32(g["x_f32_bits"])); dxq = rt.cuAlloc(K // 32 * 36)
    rt.quantize_q8_1(dx, dxq, K, 1, rt.F32)
    assert rt.from_device(dxq, (K // 32 * 36,), np.uint8).tolist() == g["xq_bytes"]
    dI, dy = rt.cuAlloc(N * (K // 32) * 4), rt.cuAlloc(N * 4)
    rt.q4k_q8_1_subdots(dW, dxq, dI, N, K)
    assert rt.from_device(dI, (N, K // 32), np.int32).tolist() == g["subdots_int32"]
    rt.gemv_q4k_q8_1(dW, dxq, dy, N, K)
    assert rt.from_device(dy, (N,), np.uint32).tolist() == g["y_f32_bits_exact_rounded_once"]
    # the batched matrix-core path returns the same bits
    dy2 = rt.cuAlloc(N * 4)
    rt.gemm_q4k_q8_1(dW, dxq, dy2, N, K, 1)
    assert rt.from_device(dy2, (N,), np.uint32).tolist() == g["y_f32_bits_exact_rounded_once"]
    for p in (dW, dx, dxq, dI, dy, dy2):
        rt.cuFree(p)


def test_argmax_gpu():
    for c in gold("argmax.json")["cases"]:
        x = argmax_input(c)
        k = rt.compileAndLoad(f"argmax VOCAB={c['V']}")
        dl, dv, di = rt.to_device(x), rt.cuAlloc(4), rt.cuAlloc(4)
        assert rt.cuLaunch(k, [1, 1, 1], [128, 1, 1], [dl, dv, di]) == 0, rt.last_error()
        rt.cuSync()
        assert int(rt.from_device(di, (1,), np.int32)[0]) == c["idx"]
        assert int(rt.from_device(dv, (1,), np.uint32)[0]) == c["val_f32_bits"]
        for p in (dl, dv, di):
            rt.cuFree(p)


def test_c_driver_reproduces_the_golden_gemv(tmp_path):
    """The compiled C caller (tests/abi/abi_driver.c: header included, library linked, no Python in between) runs
    quantize -> GEMV on the golden fixture through the typed entry points and through bk_kernel_create / bk_launch."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "abi", "abi_driver")
    assert os.path.exists(exe), "tests/abi/abi_driver is not built: make -C tests/abi"
    g = gold("gemv_q4k_q8_1.json")
    N, K = g["N"], g["K"]
    blob = tmp_path / "in.bin"
    with open(blob, "wb") as f:
        f.write(np.array([N, K], np.int32).tobytes())
        f.write(np.array(g["W_bytes"], np.uint8).tobytes())
        f.write(bits_f32(g["x_f32_bits"]).tobytes())
    r = subprocess.run([exe, str(blob)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.stdout[-400:], r.stderr[-400:])
    lines = dict(l.split(" ", 1) for l in r.stdout.strip().splitlines() if " " in l)
    assert bytes.fromhex(lines["xq"]) == bytes(g["xq_bytes"])
    want = [f"{v:08x}" for v in g["y_f32_bits_exact_rounded_once"]]
    assert lines["y"].split() == want and lines["y_launch"].split() == want
    assert [int(v, 16) - (1 << 32) if int(v, 16) >> 31 else int(v, 16) for v in lines["subdot0"].split()] == g["subdots_int32"][0]
    assert "refused" in lines and r.stdout.strip().endswith("ok")
