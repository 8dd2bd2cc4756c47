"""The fused launch's copy protocol (tickets, piece counts, flags, self-zeroing state) run on the
CPU: the copy functions are cut out of ag_matmul.hip as they are, their four device-only
statements (address-space typedefs, the LDS slot, the write-through store, the streaming load,
the wait for the memory counter)
replaced by host stand-ins, and compiled with AddressSanitizer next to a harness that runs one
host thread per GPU thread (tests/cpu/copy_protocol_harness.cpp)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE = os.path.join(ROOT, "symm-mem-recipes_amd", "csrc", "ag_matmul.hip")
HARNESS = os.path.join(ROOT, "tests", "cpu", "copy_protocol_harness.cpp")
BEGIN = "struct CopyJob {"
END = "template <int BM, int BN, bool FP8 = false>\n__global__"
STAND_INS = [
    ("typedef __attribute__((address_space(1))) u32x4 GlobalVec;", "typedef u32x4 GlobalVec;"),
    ("typedef __attribute__((address_space(3))) uint32_t LdsWord;", "typedef uint32_t LdsWord;"),
    ("reinterpret_cast<LdsWord*>((uintptr_t)lds0)", "lds_ptr(lds0)"),
    ('asm volatile("global_store_dwordx4 %0, %1, off sc1\\n\\ts_nop 1" : : "v"(dst + i), "v"(v[u]) : "memory");',
     "store_checked(dst + i, v[u]);"),
    ("__builtin_nontemporal_load(src + (i < job.chunk_vecs ? i : job.chunk_vecs - 1))",
     "load_checked(src + (i < job.chunk_vecs ? i : job.chunk_vecs - 1))"),
    ("__builtin_amdgcn_s_waitcnt(0x0F70);", ";"),
]


def _clang():
    for c in ("/opt/rocm/lib/llvm/bin/clang++", shutil.which("clang++")):
        if c and os.path.exists(c):
            return c
    return None


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    clang = _clang()
    if clang is None:
        pytest.skip("no clang++ (the copy functions use clang's vector and atomic builtins)")
    text = open(SOURCE).read()
    frag = text[text.index(BEGIN):text.index(END)]
    for old, new in STAND_INS:
        assert frag.count(old) == 1, f"the source no longer has exactly one: {old}"
        frag = frag.replace(old, new)
    assert "asm" not in frag and "__builtin_nontemporal" not in frag
    work = tmp_path_factory.mktemp("copy_protocol")
    inc = work / "fragment.inc"
    inc.write_text(frag)
    exe = work / "harness"
    subprocess.run([clang, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                    "-pthread", f'-DFRAGMENT="{inc}"', HARNESS, "-o", str(exe)], check=True, timeout=300)
    return str(exe)


# rows, 16-byte vectors per row, world_size, splits, copy-only workgroups, waiting workgroups
CASES = [
    (128, 256, 2, 1, 2, 1),     # whole pieces, both kinds of workgroup
    (256, 512, 3, 2, 3, 2),     # splits: chunk c comes from rank c / splits
    (128, 72, 2, 1, 2, 2),      # ragged: the last piece of a chunk is partial
    (384, 40, 4, 1, 3, 0),      # copy-only workgroups alone
    (384, 40, 4, 1, 0, 3),      # no copy-only workgroup at all: the waiters copy everything
    (8, 24, 2, 1, 2, 2),        # a chunk smaller than one piece
]


@pytest.mark.parametrize("case", CASES)
def test_copy_protocol_on_the_cpu(harness, case):
    r = subprocess.run([harness] + [str(x) for x in case], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.strip().endswith(": ok")
