"""The GEMM's K loop as compiled: no scratch traffic and no accumulator shuffling.

The 256x256 tiles keep 256 accumulator registers per lane next to 128 fragment
registers; whether the compiler keeps all of that in place across the loop depends on
details of code far from the loop (a changed epilogue once made it move accumulators
between register files inside the loop, 9 % slower, with every parity test green).
This test compiles the kernel to assembly (no GPU needed) and looks at the loops."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "symm-mem-recipes_amd", "csrc", "ag_matmul.hip")
HIPCC = "/opt/rocm/bin/hipcc"


def _compile(src, out):
    if not os.path.exists(HIPCC) and shutil.which("hipcc") is None:
        pytest.skip("hipcc not available")
    cmd = [HIPCC if os.path.exists(HIPCC) else "hipcc", "-O3", "-std=c++17", "--offload-arch=gfx950",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only",
           src, "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    return out.read_text()


@pytest.fixture(scope="module")
def gemm_asm(tmp_path_factory):
    return _compile(SRC, tmp_path_factory.mktemp("isa") / "ag_matmul.s")


@pytest.fixture(scope="module")
def kernels(gemm_asm):
    bodies = {}
    for m in re.finditer(r"^(_ZN3smr16ag_matmul_kernelILi(\d+)ELi(\d+)ELb([01])E\w*):[^\n]*\n(.*?)^\.Lfunc_end", gemm_asm, re.S | re.M):
        bodies[(int(m.group(2)), int(m.group(3)), m.group(4) == "1")] = m.group(5).splitlines()
    return bodies


def _k_loops(lines):
    """Innermost loops with MFMAs in them: from a label to a conditional branch back to it,
    with no other label in between."""
    labels = {}
    for i, ln in enumerate(lines):
        m = re.match(r"^(\.LBB\d+_\d+):", ln)
        if m:
            labels[m.group(1)] = i
    loops = []
    for i, ln in enumerate(lines):
        m = re.search(r"s_cbranch_\w+ (\.LBB\d+_\d+)", ln)
        if m and labels.get(m.group(1), i) < i:
            body = lines[labels[m.group(1)]:i + 1]
            if sum(bool(re.match(r"^\.LBB", x)) for x in body) == 1 and any("v_mfma_" in x for x in body):
                loops.append(body)
    return loops


@pytest.mark.parametrize("key", [(256, 256, False), (256, 256, True), (256, 128, False), (128, 128, False),
                                 (256, 128, True), (128, 128, True), (256, 224, False)])
def test_k_loop_keeps_its_registers(kernels, key):
    assert key in kernels, sorted(kernels)
    loops = _k_loops(kernels[key])
    assert loops, "K loop not found"
    # an e4m3fn loop holds two trips (one for each set of A fragments), a bf16 loop one
    trips = 2 if key[2] else 1
    for body in loops:
        text = "\n".join(body)
        mfma = len(re.findall(r"v_mfma_", text))
        assert mfma in (4, 8, 16, 32, 64, 112, 128), mfma        # whole slab pairs (112: the 256x224 tile)
        assert "scratch_" not in text, "spill inside the K loop"
        assert "v_accvgpr" not in text, "accumulators moved between register files inside the K loop"
        assert "lane_b32" not in text, "scalar registers spilled inside the K loop"
        assert re.search(r"s_waitcnt vmcnt\((8|4)\)", text), "the explicit wait for the tile loads is missing"
        assert len(re.findall(r"s_barrier", text)) == trips
        # The tile loads are assembly and waited for by hand, once per trip.  A wait of the
        # compiler's own inside the loop (it once took the copy code's piece registers for still
        # being loaded and waited where the loop first wrote one of them) drains all of them
        # every trip: the narrower kernels ran 30 % slower, every parity test green.
        waits = [i for i, x in enumerate(body) if re.search(r"s_waitcnt.*vmcnt", x)]
        by_hand = [i for i in waits if "ASMSTART" in body[i - 1]]
        assert len(by_hand) == trips and waits == by_hand, [body[i].strip() for i in waits]
        # The bf16 tile's loads leave M0 standing from one load of a slab to the next, inside
        # assembly the compiler cannot see into: nothing of the compiler's own may name M0 here.
        inside, strangers = False, []
        for x in body:
            if "ASMSTART" in x:
                inside = True
            elif "ASMEND" in x:
                inside = False
            elif not inside and re.search(r"\bm0\b", x.split(";")[0]):
                strangers.append(x.strip())
        assert not strangers, strangers


def _assembly_blocks(text):
    return re.findall(r";;#ASMSTART\n(.*?);;#ASMEND", text, re.S)


def test_assembly_stores_keep_their_data_registers(gemm_asm, tmp_path):
    """A 128-bit store written in assembly is followed, inside the same assembly block, by two idle
    slots.  The hardware reads such a store's data for two cycles after issue; the compiler keeps
    its own vector instructions away from its own stores for that long but does not look into
    assembly, and under register pressure it once reloaded a data register right behind the
    store of the fused launch's copy: one row in sixteen of the gathered operand was wrong."""
    gather_asm = _compile(os.path.join(os.path.dirname(SRC), "all_gather.hip"), tmp_path / "all_gather.s")
    stores = 0
    for text in (gemm_asm, gather_asm):
        for block in _assembly_blocks(text):
            if "global_store_dwordx4" in block or "global_store_dwordx3" in block:
                stores += 1
                lines = [x.strip() for x in block.strip().splitlines()]
                assert lines[-1].startswith("s_nop 1"), lines
    assert stores >= 2


@pytest.mark.parametrize("key", [(256, 256, True), (256, 128, True), (128, 128, True)])
def test_fp8_saturation_mode_surrounds_the_conversions_only(kernels, key):
    """The e4m3fn epilogue converts with v_cvt_pk_fp8_f32 while MODE.FP16_OVFL (bit 23) is set, and
    the MFMAs must never run with it: with the bit set they read a NaN operand as a number.  The
    conversions are intrinsics with no ordering edge to the mode write, so the compiled code is
    what is checked: in program order every conversion lies between the write that sets the bit
    and the write that clears it, and no MFMA lies in such a window."""
    assert key in kernels, sorted(kernels)
    on, conversions, windows = False, 0, 0
    for ln in kernels[key]:
        code = ln.split(";")[0]
        m = re.search(r"s_setreg_imm32_b32 hwreg\(HW_REG_MODE, 23, 1\), (\d+)", code)
        if m:
            assert on != (m.group(1) == "1"), "mode written twice the same way"
            on = m.group(1) == "1"
            windows += on
            continue
        assert not re.search(r"s_setreg", code), code.strip()        # no other mode write in the kernel
        if "v_cvt_pk_fp8_f32" in code:
            assert on, "conversion outside the saturation window"
            conversions += 1
        if "v_mfma_" in code:
            assert not on, "MFMA inside the saturation window"
    assert not on and windows >= 1 and conversions >= 16


@pytest.mark.parametrize("key", [(256, 256, False), (256, 224, False), (256, 128, False), (128, 128, False)])
def test_bf16_kernels_never_touch_the_mode_register(kernels, key):
    assert not any("s_setreg" in ln.split(";")[0] for ln in kernels[key])


def _register_counts(asm):
    """kernel name -> registers per lane a wave of it occupies (.vgpr_count of the metadata: vector
    plus accumulation registers, as allocated)."""
    out = {}
    for m in re.finditer(r"\.name:\s+(\S+)\n(?:.*\n)*?\s+\.vgpr_count:\s+(\d+)", asm):
        out[m.group(1)] = int(m.group(2))
    return out


def test_producer_fits_beside_the_gemm(gemm_asm, tmp_path):
    """smr_all_gather_beside promises workgroups that the hardware can place on a compute unit a
    GEMM workgroup already fills: one wave per SIMD, no LDS, and few enough registers that a
    GEMM wave and a producer wave fit a SIMD's 512 registers per lane together (allocation is
    in steps of 8).  True for every bf16 tile and the narrower e4m3fn ones; the 256x256 e4m3fn
    tile takes every register, which the header says."""
    gather_asm = _compile(os.path.join(os.path.dirname(SRC), "all_gather.hip"), tmp_path / "all_gather.s")
    producer = [v for k, v in _register_counts(gather_asm).items() if "all_gather_kernelILi256E" in k]
    assert len(producer) == 1
    slim = (producer[0] + 7) // 8 * 8
    gemm = {k: v for k, v in _register_counts(gemm_asm).items() if "ag_matmul_kernel" in k}
    assert len(gemm) == 7
    for name, regs in gemm.items():
        fits = (regs + 7) // 8 * 8 + slim <= 512
        if "ILi256ELi256ELb1E" in name:
            assert not fits, "the header's exception no longer holds: update include/smr.h"
        else:
            assert fits, (name, regs, slim)
