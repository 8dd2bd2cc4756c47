"""MI355X-native symmetric-memory recipes: one-shot all-reduce, blockwise barrier /
signal-pad flags, flag-gated all-gather matmul and split-K GEMV + reduce, as
hand-written HIP kernels behind the reference's Python entry points."""
from . import _lib
from .symm_mem import (EmulatedSymmetricMemory, _SymmetricMemory, _get_backend_stream,
                       enable_symm_mem_for_group, get_rank, get_world_size, set_rank,
                       set_world_size)
from .barrier import barrier_test, blockwise_barrier, send_signal, wait_signal
from .one_shot_all_reduce import one_shot_all_reduce
from .all_gather_matmul import (all_gather_matmul, all_gather_matmul_fused,
                                all_gather_matmul_tma_persistent, all_gather_with_progress,
                                gemm_schedule)
from .gemv_all_reduce import GemvWorkspace, gemv_all_reduce

__all__ = [
    "EmulatedSymmetricMemory", "_SymmetricMemory", "_get_backend_stream",
    "enable_symm_mem_for_group", "get_rank", "get_world_size", "set_rank", "set_world_size",
    "barrier_test", "blockwise_barrier", "send_signal", "wait_signal", "one_shot_all_reduce",
    "all_gather_matmul", "all_gather_matmul_fused", "all_gather_matmul_tma_persistent",
    "all_gather_with_progress", "gemm_schedule", "GemvWorkspace", "gemv_all_reduce",
]
