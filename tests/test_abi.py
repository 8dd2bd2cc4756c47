"""CPU-side checks of the C-ABI boundary: the library loads, exports every symbol
include/smr.h declares, and rejects bad arguments on the host before any launch."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "smr.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(smr_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_all_exported(lib):
    from symm_mem_recipes import _lib
    declared = _declared_symbols()
    assert len(declared) >= 15
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in smr.h but not exported"
    assert sorted(_lib.SIGNATURES) == declared, "ctypes table and header disagree"


def test_version_and_timeout_roundtrip(lib):
    assert lib.smr_version() == 111
    old = lib.smr_get_spin_timeout_us()
    assert old == 2_000_000
    assert lib.smr_set_spin_timeout_us(1234) == 0
    assert lib.smr_get_spin_timeout_us() == 1234
    assert lib.smr_set_spin_timeout_us(-5) == -1
    assert b"negative" in lib.smr_last_error_string()
    lib.smr_set_spin_timeout_us(old)


def test_reduce_grid(lib):
    assert lib.smr_reduce_num_blocks(8192, 0) == 2          # 1024 slots / 512 threads
    assert lib.smr_reduce_num_blocks(8, 0) == 1
    assert lib.smr_reduce_num_blocks(1 << 25, 0) == 256     # capped: one workgroup per compute unit
    assert lib.smr_reduce_num_blocks(0, 0) == 0
    assert lib.smr_reduce_num_blocks(4096, 1) == 2
    assert lib.smr_set_reduce_launch(256, 2048) == 0        # tuning knob
    assert lib.smr_reduce_num_blocks(1 << 25, 0) == 2048
    assert lib.smr_set_reduce_launch(100, 0) == -1
    assert lib.smr_set_reduce_launch(0, 0) == 0
    assert lib.smr_reduce_num_blocks(1 << 25, 0) == 256


def test_reduce_argument_errors_before_launch(lib):
    # every call fails validation on the host: nothing touches a GPU
    bad = lib.smr_one_shot_all_reduce
    p = 0x1000
    assert bad(p, p, p, 12, 0, 0, 8, 0, 0, None, None) == -1       # numel % 8
    assert b"128-bit aligned" in lib.smr_last_error_string()
    assert bad(p, p, p, 16, 3, 0, 8, 0, 0, None, None) == -1       # dtype
    assert bad(p, p, p, 16, 0, 8, 8, 0, 0, None, None) == -1       # rank
    assert bad(p, p, p, 16, 0, 0, 9, 0, 0, None, None) == -1       # world size
    assert bad(None, p, p, 16, 0, 0, 8, 0, 0, None, None) == -1    # null table
    assert bad(p, None, p, 16, 0, 0, 8, 0, 1, None, None) == -1    # barrier without pads
    assert bad(p, p, None, 16, 0, 0, 8, 0, 0, None, None) == -1    # no output
    assert bad(p, p, p + 4, 16, 0, 0, 8, 0, 0, None, None) == -1   # misaligned output
    assert bad(p, p, None, 16, 0, -1, 8, 1, 0, None, None) == -1   # write_all needs a rank
    assert bad(p, p, p, 0, 0, 0, 8, 0, 0, None, None) == 0         # empty message: no launch
    # the variant that takes the addresses from a host array
    by_value = lib.smr_one_shot_all_reduce_addrs
    addrs = (ctypes.c_uint64 * 8)(*[0x10000 * (r + 1) for r in range(8)])
    assert by_value(None, p, p, 16, 0, 0, 8, 0, 0, None, None) == -1
    assert by_value(addrs, p, p, 12, 0, 0, 8, 0, 0, None, None) == -1
    assert by_value(addrs, p, p, 0, 0, 0, 8, 0, 0, None, None) == 0
    addrs[5] = 0x10008                                             # not 16-byte aligned
    assert by_value(addrs, p, p, 16, 0, 0, 8, 0, 0, None, None) == -1
    assert b"16-byte aligned" in lib.smr_last_error_string()
    addrs[5] = 0
    assert by_value(addrs, p, p, 16, 0, 0, 8, 0, 0, None, None) == -1
    # the signal pads come from a host array too, and are only looked at when there is a handshake
    addrs[5] = 0x60000
    pads = (ctypes.c_uint64 * 8)(*[0x100000 * (r + 1) for r in range(8)])
    assert by_value(addrs, None, p, 16, 0, 0, 8, 0, 1, None, None) == -1
    assert b"signal pads" in lib.smr_last_error_string()
    pads[3] = 0
    assert by_value(addrs, pads, p, 16, 0, 0, 8, 0, 1, None, None) == -1
    assert b"signal pad addresses" in lib.smr_last_error_string()
    assert by_value(addrs, pads, p, 0, 0, 0, 8, 0, 1, None, None) == -1        # checked before the empty-message shortcut


def test_barrier_argument_errors(lib):
    assert lib.smr_barrier(None, 0, 8, 1, 1, 1, None, None) == -1
    assert lib.smr_barrier(0x1000, 0, 8, 0, 1, 1, None, None) == -1
    assert lib.smr_barrier(0x1000, 9, 8, 1, 1, 1, None, None) == -1
    assert lib.smr_barrier(0x1000, -1, 8, 2000, 1, 1, None, None) == -2
    assert lib.smr_signal_round(None, None, 0x1000, None, 0x1000, 0x1000, 8, 304, 24, 1, None, None) == -1
    assert lib.smr_send_signal(None, None, None) == -1
    assert lib.smr_wait_signal(None, None, None) == -1


def test_missing_library_is_loud(monkeypatch, tmp_path):
    from symm_mem_recipes import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.SmrError):
        _lib.load()


def test_knobs_set_from_two_threads_are_never_seen_half_updated(lib):
    """The launch knobs that come in pairs are one atomic word each: while one thread flips a
    pair between two settings, another thread's host-only queries see one setting or the
    other, never a mix of the two."""
    import threading
    stop = threading.Event()

    def flip():
        i = 0
        while not stop.is_set():
            if i & 1:
                lib.smr_set_reduce_launch(256, 512)
                lib.smr_set_gemv_launch(16, 2)
            else:
                lib.smr_set_reduce_launch(512, 1024)
                lib.smr_set_gemv_launch(64, 4)
            i += 1

    t = threading.Thread(target=flip)
    t.start()
    try:
        numel = 8 * 512 * 300             # 153600 slots: (256, 512) -> 512 blocks, (512, 1024) -> 300; a torn pair gives 600
        seen_reduce, seen_gemv = set(), set()
        for _ in range(20000):
            seen_reduce.add(lib.smr_reduce_num_blocks(numel, 0))
            # (16, 2): 8 * 2 senders; (64, 4): 8 * 4; the column blocks follow the same word
            seen_gemv.add((lib.smr_gemv_senders(4096, 8192, 8), ))
        assert seen_reduce <= {512, 300, 256}, seen_reduce       # 256: the default, before the first flip lands
        assert seen_gemv <= {(16,), (32,), (8,)}, seen_gemv
    finally:
        stop.set()
        t.join()
        lib.smr_set_reduce_launch(0, 0)
        lib.smr_set_gemv_launch(0, 0)
    assert lib.smr_reduce_num_blocks(1 << 25, 0) == 256


def test_fused_entry_argument_errors(lib):
    p = 0x1000
    f = lib.smr_ag_matmul_fused
    assert lib.smr_ag_matmul_fused_state_words(8, 2) == 49
    assert lib.smr_ag_matmul_fused_state_words(9, 1) == 0
    assert f(p, p, p, p, None, p, 2, 2048, 256, 256, 0, 8, 256, 0, None, None) == -1     # no state
    assert f(p, p, p, p, p, None, 2, 2048, 256, 256, 0, 8, 256, 0, None, None) == -1     # no address table
    assert f(p, p, p, p, p, p, 3, 2048, 256, 256, 0, 8, 256, 0, None, None) == -1        # element size
    assert f(p, p, p, p, p, p, 2, 2048, 256, 200, 0, 8, 256, 0, None, None) == -2        # K % 64
    assert f(p, p, p, p, p, p, 2, 2048, 256, 256, 0, 8, 256, 2000, None, None) == -1     # producer count
    assert f(p, p, p, p, p, p, 1, 2048, 256, 192, 0, 8, 256, 0, None, None) == -2        # e4m3fn: K % 128


def test_gemv_scratch_sizes_are_checked_on_the_host(lib):
    """smr_gemv_allreduce is told what the caller allocated: scratch sized under another
    setting of the launch knobs, or by an older formula, is refused before any launch."""
    p = 0x1000
    K = N = 8192
    words = lib.smr_gemv_flag_words(N, K, 8)
    senders = lib.smr_gemv_senders(N, K, 8)
    assert words == lib.smr_gemv_flag_blocks(N) * (senders + 1)
    need = senders * 4 * N * 4
    g = lib.smr_gemv_allreduce
    assert g(p, p, p, need, p, words - 1, p, 4, K, N, 8, None, None) == -1
    assert b"flag array" in lib.smr_last_error_string()
    assert g(p, p, p, need - 4, p, words, p, 4, K, N, 8, None, None) == -1
    assert b"partial sums" in lib.smr_last_error_string()
    assert g(p, p, p, need, p, lib.smr_gemv_flag_blocks(N) * senders, p, 4, K, N, 8, None, None) == -1   # the old layout


def test_device_header_is_device_only():
    """include/smr_device.h is what kernels of other libraries include: it must not need the
    library's private headers, and it declares no host function."""
    text = open(os.path.join(ROOT, "include", "smr_device.h")).read()
    includes = re.findall(r'#include\s+[<"]([^>"]+)[>"]', text)
    assert sorted(includes) == ["hip/hip_runtime.h", "smr.h", "stdint.h"], includes
    body = re.sub(r"/\*.*?\*/|//[^\n]*", "", text, flags=re.S)
    for name in ("blockwise_barrier", "send_signal", "wait_signal", "wait_signal_reset"):
        assert re.search(r"__device__ __forceinline__ \w+ " + name + r"\(", body), name
    # every function in it is a device function
    for line in body.splitlines():
        if re.match(r"^\w[\w:<> ]* \w+\(.*", line) and "constexpr" not in line and "struct" not in line:
            assert "__device__" in line, line
