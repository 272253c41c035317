"""dl_dwn_layer_fwd_static - the forward for callers that cannot allocate: its bit-plane scratch is a device
array owned by the library.  Called through the C ABI and compared with dl_dwn_layer_fwd (which takes the same
scratch as a workspace argument) on two calls in a row, the second on a smaller input, so that what the first
call left in the shared array cannot leak into the second.  Outputs and saved addresses are integer/selection
work: bit-exact.  This file is collected last on purpose (the name sorts after every other test file)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import difflut_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _run_both(lib, nat, seed, B, I, N, k, O):
    rng = np.random.default_rng(seed)
    x = torch.as_tensor(rng.random((B, I)).astype(np.float32)).to(DEV)
    idx = orc.random_mapping(I, N, k, seed=seed + 1).to(torch.int32).to(DEV).contiguous()
    luts = torch.as_tensor(rng.uniform(-1, 1, (N, O, 1 << k)).astype(np.float32)).to(DEV)
    dims = (B, I, N, k, O)
    nsaved = lib.dl_dwn_saved_bytes(*dims)
    ws = torch.empty(lib.dl_dwn_fwd_workspace_bytes(*dims), dtype=torch.uint8, device=DEV)
    y_ws = torch.full((B, N * O), float("nan"), device=DEV)
    saved_ws = torch.zeros(nsaved, dtype=torch.uint8, device=DEV)
    nat.check(lib.dl_dwn_layer_fwd(x.data_ptr(), idx.data_ptr(), luts.data_ptr(), y_ws.data_ptr(), saved_ws.data_ptr(),
                                   ws.data_ptr(), ws.numel(), *dims, nat.stream()))
    y_st = torch.full((B, N * O), float("nan"), device=DEV)
    saved_st = torch.zeros(nsaved, dtype=torch.uint8, device=DEV)
    nat.check(lib.dl_dwn_layer_fwd_static(x.data_ptr(), idx.data_ptr(), luts.data_ptr(), y_st.data_ptr(),
                                          saved_st.data_ptr(), *dims, nat.stream()))
    torch.cuda.synchronize()
    assert torch.equal(y_st, y_ws)
    if k <= 6:  # the address of every (node, row), tile-major; bytes of rows past B are unspecified in both
        BT = (B + 63) // 64
        a_st = saved_st[: BT * N * 64].view(BT, N, 64).permute(0, 2, 1).reshape(BT * 64, N)[:B]
        a_ws = saved_ws[: BT * N * 64].view(BT, N, 64).permute(0, 2, 1).reshape(BT * 64, N)[:B]
        assert torch.equal(a_st, a_ws)
    want = orc.dwn_layer_forward(x.cpu().numpy(), idx.cpu().numpy().astype(np.int64), luts.cpu().numpy())
    assert np.array_equal(y_st.cpu().numpy(), want.reshape(B, N * O))


def test_static_scratch_forward_two_calls_second_smaller():
    from difflut_amd import _native as nat
    lib = nat.lib()
    _run_both(lib, nat, 11, 700, 1000, 600, 6, 1)   # 11 batch tiles, the last one ragged
    _run_both(lib, nat, 12, 130, 52, 70, 4, 2)      # smaller in every dimension: 3 tiles, narrower planes
    _run_both(lib, nat, 13, 9, 30, 11, 7, 2)        # k > 6: the generic kernels, which use no scratch


def test_static_scratch_forward_at_its_limit_and_beyond():
    from difflut_amd import _native as nat
    lib = nat.lib()
    B, I, N, k, O = 4096, 16384, 64, 6, 1           # ceil(B/64) * I * 8 = 8 MiB: exactly the array
    _run_both(lib, nat, 14, B, I, N, k, O)
    x = torch.zeros(64, 16, device=DEV)
    one = torch.zeros(64, dtype=torch.int32, device=DEV)
    # one tile more than the array holds: refused before anything is launched
    rc = lib.dl_dwn_layer_fwd_static(x.data_ptr(), one.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(),
                                     B + 1, I, 1, 6, 1, nat.stream())
    assert rc == -6 and b"scratch" in lib.dl_error_string(rc)


def test_static_scratch_forward_allocates_nothing_and_can_be_captured():
    """After the first call on the device (which looks up the array's address) a call neither changes the device's
    free memory nor needs anything a stream capture forbids: the same call replayed from a HIP graph, with eager
    work and synchronisations in between, gives the eager result every time."""
    from difflut_amd import _native as nat
    lib = nat.lib()
    B, I, N, k, O = 300, 200, 260, 6, 1
    dims = (B, I, N, k, O)
    rng = np.random.default_rng(21)
    idx = orc.random_mapping(I, N, k, seed=22).to(torch.int32).to(DEV).contiguous()
    luts = torch.as_tensor(rng.uniform(-1, 1, (N, O, 1 << k)).astype(np.float32)).to(DEV)
    x = torch.as_tensor(rng.random((B, I)).astype(np.float32)).to(DEV)
    y = torch.empty((B, N * O), device=DEV)
    saved = torch.zeros(lib.dl_dwn_saved_bytes(*dims), dtype=torch.uint8, device=DEV)

    def call():
        nat.check(lib.dl_dwn_layer_fwd_static(x.data_ptr(), idx.data_ptr(), luts.data_ptr(), y.data_ptr(), saved.data_ptr(),
                                              *dims, nat.stream()))

    call()  # the first call on this device, outside any capture
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            call()
    for rep in range(3):
        x.copy_(torch.as_tensor(rng.random((B, I)).astype(np.float32)))
        y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        want = orc.dwn_layer_forward(x.cpu().numpy(), idx.cpu().numpy().astype(np.int64), luts.cpu().numpy())
        assert np.array_equal(y.cpu().numpy(), want.reshape(B, N * O)), rep
        assert float((y * 2).sum()) == float((y * 2).sum())  # eager work between the replays
