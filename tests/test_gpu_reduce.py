"""GPU parity of the one-shot all-reduce against the CPU oracle.
Bar: bit-exact for fp32 (rank-ordered sequential sum) and for bf16 (the kernel
accumulates in fp32 in the same order and rounds once, so it must equal the
oracle bit for bit; the stated tolerance of 1 bf16 ulp is not needed)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O

pytestmark = pytest.mark.gpu

WS = 8


def _alloc(numel, dtype, cuda, ws=WS, rank=0):
    from symm_mem_recipes import EmulatedSymmetricMemory as SM
    t = SM.empty_strided_p2p((numel,), (1,), dtype, cuda, world_size=ws, rank=rank)
    return t, SM.rendezvous(t)


def _fill(h, numel, dtype, seed0=0):
    bufs = []
    for r in range(h.world_size):
        if dtype == torch.bfloat16:
            bits = O.seeded_normal_bf16_bits(numel, seed=seed0 + r)
            h.get_buffer(r, (numel,), torch.int16).copy_(torch.from_numpy(bits.view(np.int16)))
        else:
            bits = O.seeded_normal_f32(numel, seed=seed0 + r)
            h.get_buffer(r, (numel,), torch.float32).copy_(torch.from_numpy(bits))
        bufs.append(bits)
    return bufs


def _bits(t):
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def _same(a, b):
    return np.array_equal(a.view(np.uint16 if a.dtype == np.uint16 else np.uint32),
                          b.view(np.uint16 if b.dtype == np.uint16 else np.uint32))


@pytest.fixture(autouse=True)
def _release():
    yield
    from symm_mem_recipes import EmulatedSymmetricMemory as SM
    SM.release()


def test_known_answer_ones(cuda):
    """The reference's own check (triton_one_shot_all_reduce.py:145-154)."""
    from symm_mem_recipes import one_shot_all_reduce
    t, h = _alloc(8192, torch.bfloat16, cuda)
    for r in range(WS):
        h.get_buffer(r, (8192,), torch.bfloat16).fill_(1)
    out = one_shot_all_reduce(t)
    h.check_status()
    assert out.eq(WS).all().item()
    assert out.data_ptr() != t.data_ptr() and out.dtype == torch.bfloat16
    # the pads are all-zero again after the barrier (triton_barrier.py:60-65)
    for r in range(WS):
        assert int(h.get_signal_pad(r).abs().sum().item()) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("nbytes", [16, 4096, 16 << 10, 64 << 10, (1 << 20) + 16 * 37, 2 << 20])
@pytest.mark.parametrize("barrier", [True, False])
@pytest.mark.parametrize("device_table", [False, True], ids=["addrs-by-value", "device-table"])
def test_parity_single_output(cuda, dtype, nbytes, barrier, device_table):
    """Both ways the kernel learns the peers' addresses: as kernel arguments (the default) and
    from the table in device memory, as the reference's kernel does."""
    from symm_mem_recipes import one_shot_all_reduce
    numel = nbytes // (2 if dtype == torch.bfloat16 else 4)
    t, h = _alloc(numel, dtype, cuda, rank=3)
    bufs = _fill(h, numel, dtype)
    out = one_shot_all_reduce(t, barrier=barrier, device_table=device_table)
    h.check_status()
    want = O.reduce_ref(bufs, "bf16" if dtype == torch.bfloat16 else "fp32")
    assert _same(_bits(out), want)
    # inputs untouched
    for r in range(WS):
        assert _same(_bits(h.get_buffer(r, (numel,), dtype)), bufs[r])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_parity_write_all_and_all_ranks(cuda, dtype):
    from symm_mem_recipes import one_shot_all_reduce
    numel = 3 * 8192 + 8
    t, h = _alloc(numel, dtype, cuda, rank=5)
    bufs = _fill(h, numel, dtype, seed0=20)
    want = O.reduce_ref(bufs, "bf16" if dtype == torch.bfloat16 else "fp32")
    allr = one_shot_all_reduce(t, all_ranks=True)
    h.check_status()
    assert allr.shape == (WS, numel)
    for r in range(WS):
        assert _same(_bits(allr[r]), want)
    ret = one_shot_all_reduce(t, write_all=True)
    h.check_status()
    assert ret.data_ptr() == t.data_ptr()
    for r in range(WS):
        assert _same(_bits(h.get_buffer(r, (numel,), dtype)), want)
    for r in range(WS):
        assert int(h.get_signal_pad(r).abs().sum().item()) == 0


@pytest.mark.parametrize("ws", [1, 2, 3, 4, 7])
def test_other_world_sizes(cuda, ws):
    from symm_mem_recipes import one_shot_all_reduce
    numel = 40960
    t, h = _alloc(numel, torch.bfloat16, cuda, ws=ws, rank=ws - 1)
    bufs = []
    for r in range(ws):
        bits = O.seeded_normal_bf16_bits(numel, seed=50 + r)
        h.get_buffer(r, (numel,), torch.int16).copy_(torch.from_numpy(bits.view(np.int16)))
        bufs.append(bits)
    out = one_shot_all_reduce(t)
    h.check_status()
    assert _same(_bits(out), O.reduce_ref(bufs, "bf16"))


@pytest.mark.parametrize("launch,full,held", [((64, 16), 10, 8), ((64, 4), 20, 64), ((256, 2), 70, 64), ((512, 2), 20, 8)],
                         ids=["8-held", "64-held", "64-held-twice", "512-threads"])
@pytest.mark.parametrize("mode", ["bf16", "fp32", "stepwise", "write_all", "barrier", "ws5"])
def test_results_held_back(cuda, lib, launch, full, held, mode):
    """The kernels that keep a thread's results in registers and store them in one go (8 results
    each; 64 in the kernel for workgroups of up to 256 threads with more than 16 slots per thread)
    normally run at 4 MiB per buffer and beyond.  A small grid gives a small message as many slots
    per thread: bit-exact against the oracle with a ragged last trip, every dtype and mode, behind
    the barrier (whose stand-ins share the handshake wave), and at a world size other than 8."""
    from symm_mem_recipes import one_shot_all_reduce
    threads, blocks = launch
    ws = 5 if mode == "ws5" else WS
    dtype = torch.float32 if mode == "fp32" else torch.bfloat16
    per_vec = 4 if dtype == torch.float32 else 8
    # `full` whole trips of the grid, then a ragged one: a workgroup and five threads more
    numel = (threads * blocks * full + threads + 5) * per_vec
    assert lib.smr_set_reduce_launch(threads, blocks) == 0
    try:
        slots = -(-(numel // per_vec) // (threads * blocks))
        # (the library's rule: beyond 16 slots per thread in workgroups of up to 256 threads)
        assert slots == full + 1 and (held == 64) == (threads <= 256 and slots > 16), (slots, held)
        t, h = _alloc(numel, dtype, cuda, ws=ws, rank=ws - 2)
        bufs = _fill(h, numel, dtype, seed0=70)
        print(f"held-back stores: {mode} launch {launch} numel {numel}", flush=True)
        if mode == "stepwise":
            want = O.reduce_ref_bf16_acc(bufs)
            out = one_shot_all_reduce(t, barrier=False, accumulate="bf16")
        elif mode == "write_all":
            want = O.reduce_ref(bufs, "bf16")
            one_shot_all_reduce(t, barrier=False, write_all=True)
            out = h.get_buffer(0, (numel,), dtype)
        else:
            want = O.reduce_ref(bufs, "bf16" if dtype == torch.bfloat16 else "fp32")
            out = one_shot_all_reduce(t, barrier=(mode == "barrier"))
        h.check_status()
        assert _same(_bits(out), want)
        if mode == "write_all":
            for r in range(ws):
                assert _same(_bits(h.get_buffer(r, (numel,), dtype)), want)
        if mode == "barrier":
            for r in range(ws):
                assert int(h.get_signal_pad(r).abs().sum().item()) == 0
    finally:
        lib.smr_set_reduce_launch(0, 0)


def test_special_values(cuda):
    """Signed zeros, denormals, infinities, NaN, cancellation, bf16 ties."""
    from symm_mem_recipes import one_shot_all_reduce
    numel = 64
    t, h = _alloc(numel, torch.bfloat16, cuda)
    rng = np.random.default_rng(7)
    specials = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080, 0x7F7F, 0xFF7F, 0x7F80,
                         0xFF80, 0x7FC0, 0x3F80, 0xBF80, 0x3B80, 0x4000, 0x3F81], dtype=np.uint16)
    bufs = [rng.choice(specials, size=numel).astype(np.uint16) for _ in range(WS)]
    bufs[0][:8] = 0x8000                      # all ranks -0 -> +0 (accumulator starts at +0)
    for r in range(1, WS):
        bufs[r][:8] = 0x8000
    for r in range(WS):
        h.get_buffer(r, (numel,), torch.int16).copy_(torch.from_numpy(bufs[r].view(np.int16)))
    out = _bits(one_shot_all_reduce(t))
    h.check_status()
    want = O.reduce_ref(bufs, "bf16")
    nan = np.isnan(O.bf16_bits_to_f32(want))
    assert np.array_equal(np.isnan(O.bf16_bits_to_f32(out)), nan)
    assert np.array_equal(out[~nan], want[~nan])
    assert np.all(out[:8] == 0x0000)


@pytest.mark.parametrize("numel", [8, 4096, 1 << 20])
def test_stepwise_bf16_matches_reference_chain(cuda, numel):
    """accumulate="bf16": the accumulator is rounded to bf16 after every add, as the
    reference's add.bf16x2 chain does (triton_one_shot_all_reduce.py:36-49, 84-89).
    Bar: bit-exact against the oracle's restatement of that chain."""
    from symm_mem_recipes import one_shot_all_reduce
    t, h = _alloc(numel, torch.bfloat16, cuda)
    bufs = _fill(h, numel, torch.bfloat16, seed0=40)
    out = _bits(one_shot_all_reduce(t, accumulate="bf16"))
    h.check_status()
    want = O.reduce_ref_bf16_acc(bufs)
    assert np.array_equal(out, want)
    if numel >= 4096:
        # the two accumulation modes are different functions of the same inputs
        assert not np.array_equal(want, O.reduce_ref(bufs, "bf16"))
    # write-back to all peers and all ranks in one launch share the arithmetic
    allr = _bits(one_shot_all_reduce(t, accumulate="bf16", all_ranks=True))
    h.check_status()
    assert all(np.array_equal(allr[r], want) for r in range(WS))


def test_stepwise_bf16_special_values(cuda):
    """Signed zeros, subnormals, overflow to infinity, NaN (canonical 0x7FFF), ties and
    sums whose fp32 value lies next to a bf16 rounding boundary."""
    from symm_mem_recipes import one_shot_all_reduce
    numel = 4096
    t, h = _alloc(numel, torch.bfloat16, cuda)
    rng = np.random.default_rng(11)
    specials = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080, 0x807F, 0x7F7F, 0xFF7F, 0x7F80,
                         0xFF80, 0x7FC0, 0xFFC1, 0x3F80, 0xBF80, 0x3B80, 0x4000, 0x3F81, 0x3780, 0x4B80,
                         0x3F7F, 0xBF7F, 0x0100, 0x8100], dtype=np.uint16)
    bufs = [rng.choice(specials, size=numel).astype(np.uint16) for _ in range(WS)]
    # random bit patterns too: every exponent distance between the operands occurs
    for r in range(WS):
        bufs[r][numel // 2:] = rng.integers(0, 1 << 16, numel // 2).astype(np.uint16)
        bufs[r][:8] = 0x8000                  # -0 + ... + -0 with a +0 start is +0
        h.get_buffer(r, (numel,), torch.int16).copy_(torch.from_numpy(bufs[r].view(np.int16)))
    out = _bits(one_shot_all_reduce(t, accumulate="bf16"))
    h.check_status()
    want = O.reduce_ref_bf16_acc(bufs)
    assert np.array_equal(out, want)
    assert np.all(out[:8] == 0x0000)
    assert np.any(want == 0x7FFF)


@pytest.mark.parametrize("dtype,numel", [(torch.bfloat16, 8), (torch.bfloat16, 40), (torch.bfloat16, 1 << 20),
                                         (torch.float32, 3 * 4096 + 4)])
def test_two_shot_all_reduce(cuda, dtype, numel):
    """all_ranks + write_all: rank r reduces slice r and writes it into every peer's
    buffer, between two real handshakes.  Every buffer must end up holding the
    rank-ordered sum of the original buffers, bit for bit (slices that are empty or
    ragged included: 8 bf16 = one 16-byte slot for 8 ranks)."""
    from symm_mem_recipes import one_shot_all_reduce
    t, h = _alloc(numel, dtype, cuda)
    bufs = _fill(h, numel, dtype, seed0=70)
    out = one_shot_all_reduce(t, all_ranks=True, write_all=True)
    h.check_status()
    want = O.reduce_ref(bufs, "bf16" if dtype == torch.bfloat16 else "fp32")
    assert out.shape[0] == WS
    for r in range(WS):
        assert _same(_bits(out[r]), want), r
        assert _same(_bits(h.get_buffer(r, (numel,), dtype)), want), r
    # pads are back to zero: the next collective can start
    for r in range(WS):
        assert int(h.get_signal_pad(r).abs().sum()) == 0


@pytest.mark.parametrize("write_all", [False, True])
def test_trailing_barrier(cuda, write_all):
    """A second handshake behind the last store (the reference has none): same
    result, pads self-reset after both rounds, and it can be called back to back."""
    from symm_mem_recipes import one_shot_all_reduce
    numel = 1 << 18
    t, h = _alloc(numel, torch.bfloat16, cuda)
    bufs = _fill(h, numel, torch.bfloat16, seed0=80)
    want = O.reduce_ref(bufs, "bf16")
    out = one_shot_all_reduce(t, write_all=write_all, trailing_barrier=True)
    h.check_status()
    assert _same(_bits(out), want)
    if write_all:
        for r in range(WS):
            assert _same(_bits(h.get_buffer(r, (numel,), torch.bfloat16)), want)
    else:
        for _ in range(3):
            out = one_shot_all_reduce(t, trailing_barrier=True)
        h.check_status()
        assert _same(_bits(out), want)
    for r in range(WS):
        assert int(h.get_signal_pad(r).abs().sum()) == 0


def test_validation_asserts(cuda):
    """Contract violations are AssertionErrors, as in the reference
    (triton_one_shot_all_reduce.py:102-105)."""
    from symm_mem_recipes import one_shot_all_reduce
    t, h = _alloc(8200, torch.bfloat16, cuda)
    with pytest.raises(AssertionError, match="128-bit aligned"):
        one_shot_all_reduce(t[:8196])
    with pytest.raises(AssertionError, match="supported"):
        one_shot_all_reduce(t.view(torch.int16))
    with pytest.raises(AssertionError, match="SymmetricMemory"):
        one_shot_all_reduce(torch.zeros(64, dtype=torch.bfloat16, device=cuda))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_full_size_properties_64mib(cuda, dtype):
    """Largest sweep point (64 MiB per buffer): too big to brute-force bit for
    bit in the time budget for both dtypes everywhere, so check (i) exact parity on
    three 1 MiB windows (head, unaligned middle, tail) and (ii) linearity with
    small integers over the whole message (exact, order independent)."""
    from symm_mem_recipes import one_shot_all_reduce
    nbytes = 64 << 20
    item = 2 if dtype == torch.bfloat16 else 4
    numel = nbytes // item
    t, h = _alloc(numel, dtype, cuda)
    g = torch.Generator(device=cuda).manual_seed(1)
    for r in range(WS):
        h.get_buffer(r, (numel,), dtype).copy_(
            torch.randint(-8, 9, (numel,), generator=g, device=cuda).to(dtype))
    exact = torch.zeros(numel, dtype=torch.int32, device=cuda)
    for r in range(WS):
        exact += h.get_buffer(r, (numel,), dtype).to(torch.int32)
    out = one_shot_all_reduce(t)
    h.check_status()
    assert torch.equal(out.to(torch.int32), exact)
    # windows with real-valued data
    win = (1 << 20) // item
    starts = [0, (numel // 2 + 8 * 1237) // 8 * 8, numel - win]
    bufs = {s: [] for s in starts}
    for r in range(WS):
        buf = h.get_buffer(r, (numel,), dtype)
        buf.normal_(generator=g)
        for s in starts:
            bufs[s].append(_bits(buf[s:s + win]))
    out = one_shot_all_reduce(t)
    h.check_status()
    for s in starts:
        want = O.reduce_ref(bufs[s], "bf16" if dtype == torch.bfloat16 else "fp32")
        assert _same(_bits(out[s:s + win]), want)



@pytest.mark.parametrize("form", ["write_all", "two_shot"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_write_back_forms_at_64mib(cuda, dtype, form):
    """The forms that write the sum back into all eight buffers, at the largest sweep point
    (64 MiB per buffer): (i) small integers over the whole message - exact in every order - all
    eight buffers compared with an int32 sum taken before the call; (ii) real-valued data,
    bit for bit against the oracle on three 1 MiB windows (head, unaligned middle, tail) of
    every buffer."""
    from symm_mem_recipes import one_shot_all_reduce
    nbytes = 64 << 20
    item = 2 if dtype == torch.bfloat16 else 4
    numel = nbytes // item
    t, h = _alloc(numel, dtype, cuda)
    kwargs = dict(write_all=True, all_ranks=True) if form == "two_shot" else dict(write_all=True)
    g = torch.Generator(device=cuda).manual_seed(2)
    exact = torch.zeros(numel, dtype=torch.int32, device=cuda)
    for r in range(WS):
        buf = h.get_buffer(r, (numel,), dtype)
        buf.copy_(torch.randint(-8, 9, (numel,), generator=g, device=cuda).to(dtype))
        exact += buf.to(torch.int32)
    one_shot_all_reduce(t, **kwargs)
    h.check_status()
    for r in range(WS):
        assert torch.equal(h.get_buffer(r, (numel,), dtype).to(torch.int32), exact), r
    del exact
    win = (1 << 20) // item
    starts = [0, (numel // 2 + 8 * 1237) // 8 * 8, numel - win]
    bufs = {s: [] for s in starts}
    for r in range(WS):
        buf = h.get_buffer(r, (numel,), dtype)
        buf.normal_(generator=g)
        for s in starts:
            bufs[s].append(_bits(buf[s:s + win]))
    one_shot_all_reduce(t, **kwargs)
    h.check_status()
    for s in starts:
        want = O.reduce_ref(bufs[s], "bf16" if dtype == torch.bfloat16 else "fp32")
        for r in range(WS):
            assert _same(_bits(h.get_buffer(r, (numel,), dtype)[s:s + win]), want), (s, r)
    for r in range(WS):
        assert int(h.get_signal_pad(r).abs().sum()) == 0


def test_golden_vectors(cuda):
    """The committed vectors (tests/golden/reduce.npz), independent of the oracle's code."""
    import os
    from symm_mem_recipes import one_shot_all_reduce
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reduce.npz"))
    t, h = _alloc(256, torch.bfloat16, cuda)
    for r in range(WS):
        h.get_buffer(r, (256,), torch.int16).copy_(torch.from_numpy(g["bf16_in"][r].view(np.int16)))
    assert np.array_equal(_bits(one_shot_all_reduce(t)), g["bf16_out"])
    assert np.array_equal(_bits(one_shot_all_reduce(t, accumulate="bf16")), g["bf16_out_bf16_acc"])
    t, h = _alloc(256, torch.float32, cuda)
    for r in range(WS):
        h.get_buffer(r, (256,), torch.float32).copy_(torch.from_numpy(g["fp32_in"][r]))
    assert np.array_equal(_bits(one_shot_all_reduce(t)).view(np.uint32), g["fp32_out"].view(np.uint32))
    h.check_status()


@pytest.mark.parametrize("barrier", [False, True])
def test_reduce_replays_from_a_graph(cuda, barrier):
    """Launches captured into a HIP graph (kernel nodes only) give the eager bits on every
    replay, with eager work and synchronisations between the replays; with the barrier the
    signal pads must come back to zero after each replay for the next one to pass."""
    from symm_mem_recipes import one_shot_all_reduce
    numel = 1 << 18
    t, h = _alloc(numel, torch.bfloat16, cuda)
    bufs = _fill(h, numel, torch.bfloat16, seed0=11)
    want = O.reduce_ref(bufs, "bf16")
    eager = one_shot_all_reduce(t, barrier=barrier)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(eager), want)
    side = torch.cuda.Stream(cuda)
    side.wait_stream(torch.cuda.current_stream(cuda))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            outs = [one_shot_all_reduce(t, barrier=barrier) for _ in range(3)]
    torch.cuda.current_stream(cuda).wait_stream(side)
    for replay in range(4):
        for o in outs:
            o.zero_()
        noise = torch.randn(1 << 18, device=cuda).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        h.check_status()
        for o in outs:
            assert np.array_equal(_bits(o), want), replay
        del noise
    del graph
