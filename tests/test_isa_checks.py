"""Properties of the compiled gfx950 code that the source relies on but the compiler does not guarantee (CPU only: hipcc
cross-compiles without a GPU).

attn_exact.hip issues v_fmac_f64 with a DPP operand from inline assembly.  The compiler's hazard recognizer does not look
into asm blocks, so the idle cycles a DPP read needs are written by hand (two, in front of every group, against a vector
write of the DPP source) or avoided by construction (five behind a vector instruction that writes EXEC: the kernel must
not contain one)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "bunker_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _compile_to_asm(tmp_path_factory, source):
    if not (os.path.exists(HIPCC) or shutil.which(HIPCC)):
        pytest.skip("hipcc not found")
    out = str(tmp_path_factory.mktemp("isa") / (source + ".s"))
    flags = re.search(r"^HIPFLAGS \?= (.*?)(?<!\\)$", open(os.path.join(CSRC, "Makefile")).read(), flags=re.M | re.S).group(1)
    flags = flags.replace("\\\n", " ").replace("$(ARCH)", "gfx950").split()
    subprocess.check_call([HIPCC, *flags, "-S", "--cuda-device-only", "-o", out, os.path.join(CSRC, source)],
                          stderr=subprocess.DEVNULL)
    return open(out).read()


@pytest.fixture(scope="module")
def exact_asm(tmp_path_factory):
    return _compile_to_asm(tmp_path_factory, "attn_exact.hip")


def _kernels(asm):
    """name -> body of every kernel of the file"""
    out = {}
    for m in re.finditer(r"^(_ZN2bk\w+):[^\n]*\n(.*?)^\.Lfunc_end", asm, flags=re.M | re.S):
        out[m.group(1)] = m.group(2)
    return out


def test_dpp_groups_in_the_exact_attention_are_hazard_free(exact_asm):
    ks = {k: v for k, v in _kernels(exact_asm).items() if "attn_exact_kernel" in k}
    assert len(ks) == 4                                         # plain / nontemporal loads x with / without the folded preparation
    for name, body in ks.items():
        n_dpp = len(re.findall(r"\bv_fmac_f64_dpp\b", body))
        assert n_dpp >= 512 and n_dpp % 8 == 0, (name, n_dpp)
        # no vector instruction writes EXEC anywhere in the kernel
        assert not re.search(r"\bv_cmpx", body), name
        # every DPP instruction sits in an asm block that opens with the two idle cycles, eight to a block
        blocks = re.findall(r";;#ASMSTART\n(.*?);;#ASMEND", body, flags=re.S)
        dpp_blocks = [b for b in blocks if "v_fmac_f64_dpp" in b]
        assert sum(len(re.findall(r"v_fmac_f64_dpp", b)) for b in dpp_blocks) == n_dpp
        for b in dpp_blocks:
            lines = [l.strip() for l in b.strip().splitlines()]
            assert lines[0] == "s_nop 1" and len(lines) == 9 and all(l.startswith("v_fmac_f64_dpp") for l in lines[1:]), b
            # the broadcast source is read, never written, inside the block
            src = {re.match(r"v_fmac_f64_dpp (v\[\d+:\d+\]), (v\[\d+:\d+\]),", l).group(2) for l in lines[1:]}
            dst = {re.match(r"v_fmac_f64_dpp (v\[\d+:\d+\]),", l).group(1) for l in lines[1:]}
            assert len(src) == 1 and not (src & dst), b
        # no register spills: the kernel is sized for 128 registers per lane and 4 waves per SIMD
        meta = re.search(r"\.name:\s+%s\n(.*?)\.wavefront_size" % re.escape(name), exact_asm, flags=re.S).group(1)
        assert int(re.search(r"\.vgpr_count:\s+(\d+)", meta).group(1)) <= 128
        assert int(re.search(r"\.vgpr_spill_count:\s+(\d+)", meta).group(1)) == 0


@pytest.mark.parametrize("source,kernels,transfer,mfma,min_mfma", [
    ("attn_prefill.hip", ["attn_prefill_kernel"], "global_load_lds_dwordx4", "v_mfma_f32_32x32x16_bf16", 64),
    ("gdn_chunk.hip", ["gdn_chunk_wu_kernel", "gdn_chunk_state_kernel", "gdn_chunk_out_kernel"], "global_load_lds_dword", "v_mfma_f32_32x32x2_f32", 32),
])
def test_lds_transfers_written_as_instructions_own_m0(tmp_path_factory, source, kernels, transfer, mfma, min_mfma):
    """lds_dma16 / lds_dma4 (common.h) set m0 themselves and tell the compiler so, but m0 is a register the compiler
    reserves: the kernels that use them must contain no other use of it, every write of m0 must be followed (one idle
    cycle later) by the transfer that reads it, and the compiler's own form of the transfer — behind which it waits for
    the whole transfer before the next LDS access — must not have come back.  Also: no vector spills, no scalar spills
    in the blocks that issue matrix instructions, no scratch, and the matrix instruction the kernel is built around is
    there."""
    asm = _compile_to_asm(tmp_path_factory, source)
    bodies = _kernels(asm)
    for kname in kernels:
        name, body = next((k, v) for k, v in bodies.items() if kname in k)
        lines = [l.strip() for l in body.split("\n") if l.strip() and not l.strip().startswith((";", "."))]
        m0 = [i for i, l in enumerate(lines) if re.search(r"\bm0\b", l)]
        assert m0, name
        for i in m0:
            assert lines[i].startswith("s_mov_b32 m0,"), (name, lines[i])
            assert lines[i + 1].startswith("s_nop") and lines[i + 2].startswith(transfer + " "), (name, lines[i:i + 3])
        assert sum(l.startswith(transfer + " ") for l in lines) == len(m0), name
        assert sum(l.startswith(mfma + " ") for l in lines) >= min_mfma, name
        meta = re.search(r"\.name:\s+%s\n(.*?)\.wavefront_size" % re.escape(name), asm, flags=re.S).group(1)
        assert int(re.search(r"\.vgpr_spill_count:\s+(\d+)", meta).group(1)) == 0, name
        # scalar registers: a handful of spills in the set-up code are tolerated, none where matrix instructions are issued
        # (a spilled scalar is a lane read or write in the wave's instruction stream)
        assert int(re.search(r"\.sgpr_spill_count:\s+(\d+)", meta).group(1)) <= 8, name
        for block in re.split(r"^\.LBB\d+_\d+:", body, flags=re.M):
            if block.count(mfma + " ") >= 4:
                assert "v_readlane_b32" not in block and "v_writelane_b32" not in block, name
        assert int(re.search(r"\.private_segment_fixed_size:\s+(\d+)", meta).group(1)) == 0, name


@pytest.mark.parametrize("source,kernel,kernarg_sizes", [
    # SwiGLU pair 52 (padded to 56), one matrix 64, several matrices 104 / 128 with the convolution's operands, general
    # 176 / 208; no implicit arguments behind them (the kernel reads the grid size from its block, not from gridDim)
    ("gemv_fused.hip", "gemv_fused_kernel", {56, 64, 104, 128, 176, 208}),
    ("gdn.hip", "gdn_slab_kernel", {80}),
    ("gemm_mfma.hip", "gemm_q4k_q8_1_mfma_kernel", {56, 64, 184}),
])
def test_argument_blocks_stay_compact_and_in_registers(tmp_path_factory, source, kernel, kernarg_sizes):
    """The decode step's kernels take the smallest by-value argument block their form needs (a launch pays for every
    64-byte line of it) and rebuild the general block in registers.  That only works while the compiler keeps the rebuilt
    block out of private memory and LDS: no kernel of these families may have a private segment, and every argument-block
    size the launchers rely on must be there."""
    asm = _compile_to_asm(tmp_path_factory, source)
    seen = set()
    for m in re.finditer(r"\.kernarg_segment_size:\s+(\d+)\n(.*?)\.name:\s+(\S+)\n(.*?)\.wavefront_size", asm, flags=re.S):
        if kernel not in m.group(3):
            continue
        meta = m.group(2) + m.group(4)
        seen.add(int(m.group(1)))
        assert int(re.search(r"\.private_segment_fixed_size:\s+(\d+)", meta).group(1)) == 0, m.group(3)
        assert int(re.search(r"\.vgpr_spill_count:\s+(\d+)", meta).group(1)) == 0, m.group(3)
    assert seen and seen <= kernarg_sizes and min(seen) == min(kernarg_sizes), seen
