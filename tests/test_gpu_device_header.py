"""The public device header (include/smr_device.h) used from a kernel library that is not part
of the package: tests/device_header/flag_client.hip is compiled against include/ only and links
nothing of libsmr_gfx950.so.  The signal pads it runs on are the emulated handle's."""
import ctypes
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
CLIENT = os.path.join(HERE, "device_header", "libflag_client.so")


@pytest.fixture(scope="module")
def client():
    if not os.path.exists(CLIENT):
        pytest.fail(f"{CLIENT} is missing: build it with `make -C tests/device_header`")
    lib = ctypes.CDLL(CLIENT)
    p, i, u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64
    lib.client_barrier_rounds.restype = i
    lib.client_barrier_rounds.argtypes = [p, p, p, i, i, i, u64, p, p]
    lib.client_send_then_wait.restype = i
    lib.client_send_then_wait.argtypes = [p, p, ctypes.c_uint32, p, u64, p, p, p]
    return lib


@pytest.fixture
def handle(cuda):
    from symm_mem_recipes import EmulatedSymmetricMemory as SM
    t = SM.empty_strided_p2p((1024,), (1,), torch.int32, cuda, world_size=8)
    yield SM.rendezvous(t)
    SM.release()


@pytest.mark.parametrize("ws,blocks,rounds", [(8, 32, 200), (8, 304, 50), (3, 5, 20)])
def test_client_kernel_runs_the_barrier_with_a_payload(client, cuda, ws, blocks, rounds):
    """blockwise_barrier from the header in a foreign kernel: every round each workgroup sees
    what its partners wrote before their call (plain stores, published and acquired by the
    barrier), the pads are zero again afterwards."""
    from symm_mem_recipes import EmulatedSymmetricMemory as SM
    t = SM.empty_strided_p2p((1024,), (1,), torch.int32, cuda, world_size=ws)
    h = SM.rendezvous(t)
    words = torch.zeros(2 * ws * blocks, dtype=torch.int32, device=cuda)
    bad = torch.zeros(1, dtype=torch.int32, device=cuda)
    print(f"client barrier: ws {ws} blocks {blocks} rounds {rounds}", flush=True)
    rc = client.client_barrier_rounds(h.signal_pad_ptrs_dev, words.data_ptr(), bad.data_ptr(), ws, blocks, rounds,
                                      200_000_000, h.status.data_ptr(), torch.cuda.current_stream(cuda).cuda_stream)
    assert rc == 0
    h.check_status()
    assert int(bad.item()) == 0
    for r in range(ws):
        assert int(h.get_signal_pad(r).abs().sum().item()) == 0
    SM.release()


def test_client_kernels_send_and_wait(client, cuda, handle):
    """send_signal / wait_signal / wait_signal_reset from the header: the waiter, launched first
    on its own stream, sees the payload the sender wrote before raising the flag, and leaves the
    flag consumed."""
    pad = handle.get_signal_pad(0)
    flag_addr = pad.data_ptr() + 64
    payload = torch.zeros(1, dtype=torch.int32, device=cuda)
    out = torch.zeros(64, dtype=torch.int32, device=cuda)
    torch.cuda.synchronize()
    waiter, sender = torch.cuda.Stream(cuda), torch.cuda.Stream(cuda)
    rc = client.client_send_then_wait(flag_addr, payload.data_ptr(), 0x5EED, out.data_ptr(), 200_000_000,
                                      handle.status.data_ptr(), sender.cuda_stream, waiter.cuda_stream)
    assert rc == 0
    waiter.synchronize()
    sender.synchronize()
    handle.check_status()
    assert out.cpu().tolist() == [0x5EED] * 64
    assert int(pad.abs().sum().item()) == 0
