"""ctypes binding of libsmr_gfx950.so (the C ABI declared in include/smr.h).

The library is loaded, never built, from this directory; a missing library is a
hard error - there is no fallback path of any kind.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

LIB_NAME = "libsmr_gfx950.so"
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

DTYPE_BF16 = 0
DTYPE_FP32 = 1
DTYPE_BF16_STEPWISE = 2
BARRIER_NONE = 0
BARRIER_PROXY = 1
BARRIER_BOTH = 2
STATUS_WORDS = 4
MAX_WORLD_SIZE = 8

ST_OK, ST_SEND_TIMEOUT, ST_WAIT_TIMEOUT, ST_MISMATCH = 0, 1, 2, 3
STATUS_TEXT = {
    ST_SEND_TIMEOUT: "send_signal timed out (slot never returned to 0)",
    ST_WAIT_TIMEOUT: "wait_signal timed out (flag never arrived)",
    ST_MISMATCH: "signal-round checksum mismatch",
}

_p, _i, _i64, _u32 = C.c_void_p, C.c_int, C.c_int64, C.c_uint32

# name -> (restype, argtypes); mirrors include/smr.h one to one
SIGNATURES = {
    "smr_version": (_i, []),
    "smr_last_error_string": (C.c_char_p, []),
    "smr_set_spin_timeout_us": (_i, [_i64]),
    "smr_get_spin_timeout_us": (_i64, []),
    "smr_set_trace_buffer": (_i, [_p, _i64]),
    "smr_one_shot_all_reduce": (_i, [_p, _p, _p, _i64, _i, _i, _i, _i, _i, _p, _p]),
    "smr_one_shot_all_reduce_addrs": (_i, [_p, _p, _p, _i64, _i, _i, _i, _i, _i, _p, _p]),
    "smr_reduce_num_blocks": (_i, [_i64, _i]),
    "smr_set_reduce_launch": (_i, [_i, _i]),
    "smr_barrier": (_i, [_p, _i, _i, _i, _i, _i, _p, _p]),
    "smr_send_signal": (_i, [_p, _p, _p]),
    "smr_wait_signal": (_i, [_p, _p, _p]),
    "smr_wait_signal_reset": (_i, [_p, _p, _p]),
    "smr_stream_write_value32": (_i, [_p, _u32, _p]),
    "smr_signal_round": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i64, _i, _p, _p]),
    "smr_all_gather_with_progress": (_i, [_p, _p, _p, _p, _i, _i, _i64, _i, _i, _p]),
    "smr_all_gather_at_once": (_i, [_p, _p, _p, _p, _i, _i, _i64, _i, _i, _p]),
    "smr_all_gather_beside": (_i, [_p, _p, _p, _p, _i, _i, _i64, _i, _i, _i64, _i, _p]),
    "smr_ag_matmul_pace": (_i, [_i, _i, _i, _i, _i, _i, _p]),
    "smr_set_ag_matmul_acquire": (_i, [_i]),
    "smr_ag_matmul_fused": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p, _p]),
    "smr_ag_matmul_fused_state_words": (_i, [_i, _i]),
    "smr_ag_matmul": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _p]),
    "smr_ag_matmul_schedule": (_i, [_i, _i, _i, _i, _i, _i, _i, _p, _i]),
    "smr_ag_matmul_grid": (_i, [_i, _i, _i, _i, _i, _i]),
    "smr_set_ag_matmul_grid_limit": (_i, [_i]),
    "smr_ag_matmul_plan": (_i, [_i, _i, _i, _i, _i, _p]),
    "smr_ag_matmul_fp8": (_i, [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _p]),
    "smr_ag_matmul_plan_fp8": (_i, [_i, _i, _i, _i, _i, _p]),
    "smr_gemv_allreduce": (_i, [_p, _p, _p, _i64, _p, _i64, _p, _i, _i, _i, _i, _p, _p]),
    "smr_gemv_allreduce_static": (_i, [_p, _p, _p, _i, _i, _i, _i, _p, _p]),
    "smr_gemv_static_scratch_bytes": (_i64, []),
    "smr_gemv_flag_blocks": (_i, [_i]),
    "smr_gemv_senders": (_i, [_i, _i, _i]),
    "smr_gemv_flag_words": (_i, [_i, _i, _i]),
    "smr_set_gemv_launch": (_i, [_i, _i]),
    "smr_set_gemv_matrix_cores": (_i, [_i]),
}

_lib: Optional[C.CDLL] = None
_probe: Optional[C.CDLL] = None

PROBE_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libsmr_probe.so")


def load_probe() -> C.CDLL:
    """libsmr_probe.so: the MFMA-only measurement kernel (csrc/probe/mfma_probe.hip), a library
    of its own that only the benchmark and its test load - no part of the C ABI."""
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_PATH):
            raise SmrError(f"{PROBE_PATH} is missing: build it with `make -C symm-mem-recipes_amd/csrc`")
        _probe = C.CDLL(PROBE_PATH)
        _probe.smr_probe_mfma_only.restype = _i
        _probe.smr_probe_mfma_only.argtypes = [_p, _i, _i, _i, _p, _p, _p]
    return _probe


class SmrError(RuntimeError):
    pass


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise SmrError(
            f"{LIB_PATH} is missing: build it with `make -C symm-mem-recipes_amd/csrc` "
            "(hipcc, gfx950). There is no fallback implementation.")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    """Raise on a non-zero return code.  Argument errors become AssertionError, the
    reference's convention for contract violations
    (symm_mem_recipes/triton_one_shot_all_reduce.py:102-105)."""
    if code == 0:
        return
    msg = load().smr_last_error_string().decode("utf-8", "replace")
    if code in (-1, -2):
        raise AssertionError(f"{what}: {msg}")
    raise SmrError(f"{what}: error {code}: {msg}")
