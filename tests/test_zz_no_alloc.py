"""The entry point that allocates nothing, smr_gemv_allreduce_static, against the entry point
it is a variant of, smr_gemv_allreduce, through the C ABI: same kernels, so the bf16 results
must be identical bit for bit; and against the CPU oracle, to the GEMV's bar.  Two calls in a
row share the library's one scratch array, the second with a smaller input; every buffer is
allocated before the calls under test, and the device's free memory and torch's allocation
count are the same after them as before."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _bits_t(bits):
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def _case(lib, cuda, batch, K, N, ws, seed):
    x = _bits_t(O.seeded_normal_bf16_bits(batch * K, seed=seed).reshape(batch, K)).to(cuda)
    w = _bits_t(O.seeded_normal_bf16_bits(K * N, seed=seed + 1, std=0.02).reshape(K, N)).to(cuda)
    senders = lib.smr_gemv_senders(N, K, ws)
    partials = torch.empty(senders, batch, N, dtype=torch.float32, device=cuda)
    flags = torch.zeros(lib.smr_gemv_flag_words(N, K, ws), dtype=torch.int32, device=cuda)
    want = torch.empty(batch, N, dtype=torch.bfloat16, device=cuda)
    got = torch.full((batch, N), float("nan"), dtype=torch.bfloat16, device=cuda)
    status = torch.zeros(4, dtype=torch.int32, device=cuda)
    oracle = O.gemv_allreduce_ref(O.seeded_normal_bf16_bits(batch * K, seed=seed).reshape(batch, K),
                                  O.seeded_normal_bf16_bits(K * N, seed=seed + 1, std=0.02).reshape(K, N), ws)
    return dict(x=x, w=w, partials=partials, flags=flags, want=want, got=got, status=status,
                shape=(batch, K, N, ws), oracle=oracle)


def test_static_scratch_entry_matches_the_workspace_entry(lib, cuda):
    stream = torch.cuda.current_stream(cuda).cuda_stream
    assert lib.smr_gemv_static_scratch_bytes() == 4 << 20
    # the second case is smaller in every dimension: it reuses the front of the array the first left behind
    cases = [_case(lib, cuda, 8, 8192, 8192, 8, seed=10), _case(lib, cuda, 3, 1024, 1000, 4, seed=20)]
    torch.cuda.synchronize()
    for c in cases:
        batch, K, N, ws = c["shape"]
        print(f"gemv static: batch {batch} K {K} N {N} ws {ws}", flush=True)
        rc = lib.smr_gemv_allreduce(c["x"].data_ptr(), c["w"].data_ptr(), c["partials"].data_ptr(),
                                    c["partials"].numel() * 4, c["flags"].data_ptr(), c["flags"].numel(),
                                    c["want"].data_ptr(), batch, K, N, ws, c["status"].data_ptr(), stream)
        assert rc == 0, lib.smr_last_error_string()
    # the first static call of the process looks the array's address up (no allocation either,
    # but the runtime may load the code object's data lazily): take the snapshot behind one call
    c = cases[1]
    batch, K, N, ws = c["shape"]
    assert lib.smr_gemv_allreduce_static(c["x"].data_ptr(), c["w"].data_ptr(), c["got"].data_ptr(),
                                         batch, K, N, ws, c["status"].data_ptr(), stream) == 0
    torch.cuda.synchronize()
    c["got"].fill_(float("nan"))
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(cuda)
    allocated_before = torch.cuda.memory_allocated(cuda)
    reserved_before = torch.cuda.memory_reserved(cuda)
    for c in cases:                                   # back to back, nothing in between
        batch, K, N, ws = c["shape"]
        rc = lib.smr_gemv_allreduce_static(c["x"].data_ptr(), c["w"].data_ptr(), c["got"].data_ptr(),
                                           batch, K, N, ws, c["status"].data_ptr(), stream)
        assert rc == 0, lib.smr_last_error_string()
    torch.cuda.synchronize()
    # nothing was allocated: not by torch, not behind its back
    assert torch.cuda.memory_allocated(cuda) == allocated_before
    assert torch.cuda.memory_reserved(cuda) == reserved_before
    assert torch.cuda.mem_get_info(cuda)[0] == free_before
    for c in cases:
        assert c["status"].cpu().tolist() == [0, 0, 0, 0]
        assert torch.equal(c["got"].view(torch.int16), c["want"].view(torch.int16))
        # and the oracle, to the GEMV's bar: 1e-2 relative, with the result's scale for entries near zero
        got = O.bf16_bits_to_f32(c["got"].view(torch.int16).cpu().numpy().view(np.uint16)).astype(np.float64)
        ref = O.bf16_bits_to_f32(c["oracle"]).astype(np.float64)
        rms = float(np.sqrt(np.mean(ref ** 2)))
        assert np.all(np.abs(got - ref) <= 1e-2 * np.abs(ref) + 1e-2 * rms)
    # a third call, the large case again after the small one
    c = cases[0]
    c["got"].fill_(float("nan"))
    batch, K, N, ws = c["shape"]
    rc = lib.smr_gemv_allreduce_static(c["x"].data_ptr(), c["w"].data_ptr(), c["got"].data_ptr(),
                                       batch, K, N, ws, c["status"].data_ptr(), stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(c["got"].view(torch.int16), c["want"].view(torch.int16))


def test_static_scratch_entry_rejects_what_does_not_fit(lib, cuda):
    stream = torch.cuda.current_stream(cuda).cuda_stream
    # 8 senders x 8 rows x 32768 columns x 4 B = 8 MiB of partial sums: beyond the 4 MiB array
    batch, K, N, ws = 8, 64, 32768, 8
    x = torch.zeros(batch, K, dtype=torch.bfloat16, device=cuda)
    w = torch.zeros(K, N, dtype=torch.bfloat16, device=cuda)
    out = torch.zeros(batch, N, dtype=torch.bfloat16, device=cuda)
    rc = lib.smr_gemv_allreduce_static(x.data_ptr(), w.data_ptr(), out.data_ptr(), batch, K, N, ws, None, stream)
    assert rc == -2
    assert b"partial sums" in lib.smr_last_error_string()
    assert lib.smr_gemv_allreduce_static(None, w.data_ptr(), out.data_ptr(), 1, K, 64, ws, None, stream) == -1
    torch.cuda.synchronize()
