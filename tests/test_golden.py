"""The CPU checker against the committed known-answer fixtures of tests/golden/ (written by
tests/golden/make_golden.py from integer / exact-rational restatements of the reference's rules;
neither the checker nor the kernels produced them)."""
import json
import os

import numpy as np

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def gold(name):
    with open(os.path.join(GOLD, name)) as f:
        return json.load(f)


def bits_f32(bits):
    return np.asarray(bits, np.uint32).view(np.float32)


def argmax_input(case):
    V = case["V"]
    if case["fill"] == "zeros":
        x = np.zeros(V, np.float32)
    else:
        x = (np.sin(np.arange(V, dtype=np.float64)) * 10).astype(np.float32)
    for k, v in case["overrides"].items():
        x[int(k)] = v
    return x


def test_fp16_encode(orc):
    for c in gold("fp16_encode.json")["cases"]:
        v = float(bits_f32([c["f32_bits"]])[0])
        assert orc.encode_half(v) == c["half_bits"], c
        if v != 0.0:        # src/kernel.ts:16-32 works on the bits and keeps the sign of -0; bench.ts:41-51 returns 0 for both zeros
            assert int(orc.f32to16(np.array([v], np.float32))[0]) == c["half_bits"], c


def test_q8_1_blocks(orc):
    for b in gold("q8_1_blocks.json")["blocks"]:
        got = orc.pack_q8_1(bits_f32(b["x_f32_bits"]))
        assert got[:32].view(np.int8).tolist() == b["q"]
        assert int(got[32:34].view(np.uint16)[0]) == b["d_half_bits"] and int(got[34:36].view(np.uint16)[0]) == b["s_half_bits"]


def test_legacy_dequant(orc):
    for b in gold("legacy_dequant.json")["blocks"]:
        assert orc.legacy_dequant_i8(np.array(b["block_bytes"], np.uint8)).tolist() == b["int8"]


def test_q4k_block(orc):
    g = gold("q4k_block.json")
    blk = np.array(g["block_bytes"], np.uint8)
    sc, m = orc.q4k_unpack_scales(blk[4:16])
    assert sc.tolist() == g["scales"] and m.tolist() == g["mins"]
    assert orc.q4k_pack_scales(sc, m).tolist() == blk[4:16].tolist()
    assert orc.q4k_nibbles(blk).tolist() == g["nibbles"]
    # the checker forms d*sc*nib and dmin*m in f32 and subtracts: within one ulp of the exactly rounded value
    w = orc.q4k_dequant(blk)
    ref = bits_f32(g["w_f32_bits_exact_rounded_once"])
    assert np.all(np.abs(w.astype(np.float64) - ref) <= np.spacing(np.abs(ref)).astype(np.float64) * 2)


def test_gemv_q4k_q8_1(orc):
    g = gold("gemv_q4k_q8_1.json")
    N, K = g["N"], g["K"]
    W = np.array(g["W_bytes"], np.uint8)
    xq = orc.pack_q8_1(bits_f32(g["x_f32_bits"]))
    assert xq.tolist() == g["xq_bytes"]
    assert orc.q4k_q8_1_subdots(W, xq, N, K).tolist() == g["subdots_int32"]
    y = orc.gemv_q4k_q8_1(W, xq, N, K)
    assert y.view(np.uint32).tolist() == g["y_f32_bits_exact_rounded_once"]


def test_argmax(orc):
    for c in gold("argmax.json")["cases"]:
        v, i = orc.argmax(argmax_input(c))
        assert i == c["idx"] and np.float32(v).view(np.uint32) == c["val_f32_bits"], c
