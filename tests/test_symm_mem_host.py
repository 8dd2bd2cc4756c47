"""Host logic of the emulated symmetric-memory handle, on CPU tensors (the handle
itself never launches anything)."""
import pytest
import torch

from symm_mem_recipes import EmulatedSymmetricMemory as SM, set_rank, get_rank


@pytest.fixture(autouse=True)
def _clean():
    yield
    SM.release()
    set_rank(0)


def test_views_pointer_tables_and_rendezvous():
    t = SM.empty_strided_p2p((4, 16), (16, 1), torch.bfloat16, "cpu", world_size=8, rank=3)
    h = SM.rendezvous(t)
    assert h is not None and h.rank == 3 and h.world_size == 8
    assert t.shape == (4, 16) and t.data_ptr() == h.buffer_ptrs[3]
    for r in range(8):
        v = h.get_buffer(r, (4, 16), torch.bfloat16)
        assert v.data_ptr() == h.buffer_ptrs[r]
        v.fill_(r)
    for r in range(8):                                   # no aliasing between ranks
        assert h.get_buffer(r, (64,), torch.bfloat16).eq(r).all()
    off = h.get_buffer(2, (2, 16), torch.bfloat16, 32)   # storage_offset in elements
    assert off.data_ptr() == h.buffer_ptrs[2] + 64
    assert h._group.buffer_ptrs.tolist() == h.buffer_ptrs
    assert h._group.pad_ptrs.tolist() == h.signal_pad_ptrs
    assert h.get_signal_pad(5).data_ptr() == h.signal_pad_ptrs[5]
    assert int(h.get_signal_pad(0).abs().sum()) == 0      # pads start zeroed
    assert h.signal_pad_size >= 304 * 8 * 4               # room for 304 blocks x 8 ranks
    assert SM.rendezvous(torch.zeros(4)) is None
    other = h.for_rank(6)
    assert other.rank == 6 and other.buffer_ptrs_dev == h.buffer_ptrs_dev
    with pytest.raises(AssertionError):
        h.get_buffer(0, (4, 64), torch.bfloat16)          # larger than the allocation


def test_rank_selection_and_release():
    set_rank(5)
    assert get_rank() == 5
    t = SM.empty_strided_p2p((8,), (1,), torch.float32, "cpu", world_size=8)
    assert SM.rendezvous(t).rank == 5
    SM.release(t)
    assert SM.rendezvous(t) is None
    with pytest.raises(AssertionError):
        SM.empty_strided_p2p((8,), (1,), torch.float32, "cpu", world_size=9)


def test_reference_import_paths_resolve():
    """A caller written against the reference's module names gets the same functions."""
    import importlib
    import symm_mem_recipes as pkg
    for module, names in (("triton_one_shot_all_reduce", ("one_shot_all_reduce",)),
                          ("triton_barrier", ("barrier_test", "blockwise_barrier")),
                          ("triton_all_gather_matmul", ("all_gather_with_progress", "all_gather_matmul",
                                                        "all_gather_matmul_tma_persistent")),
                          ("utils", ("benchmark_with_event", "benchmark_with_profiler"))):
        mod = importlib.import_module(f"symm_mem_recipes.{module}")
        for name in names:
            assert callable(getattr(mod, name))
            if hasattr(pkg, name):
                assert getattr(mod, name) is getattr(pkg, name)
