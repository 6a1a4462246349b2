"""GPU test of the tzgemm entry point that allocates nothing (its workspace is a static device
array of the library): output against tacker_gptb_tzgemm's, bit for bit, on calls in a row that
share the array, the later ones with smaller inputs; no tkMalloc / tkFree and no change of the
device's free memory around the call; and the call recorded into a HIP graph and replayed."""
import ctypes as C

import numpy as np
import pytest
import torch

import tacker_amd as ta
from gpu_util import dev, gemm_inputs, host, setup

pytestmark = pytest.mark.gpu


def both(M, N, K, seed, tile_start=0, tile_end=None):
    A, B = gemm_inputs(M, N, K, seed)
    dA, dB = dev(A), dev(B)
    want = torch.full((M, N), -7.0, device="cuda:0")
    got = torch.full((M, N), -7.0, device="cuda:0")
    ta.gptb_tzgemm(dA, dB, want, tile_start, tile_end)
    torch.cuda.synchronize()
    # three witnesses: the library's own count of tkMalloc / tkFree calls (every device allocation
    # of the library goes through them), the driver's free memory, torch's caching allocator
    calls = ta.allocation_calls()
    free_bytes = torch.cuda.mem_get_info()[0]
    before = torch.cuda.memory_allocated()
    ta.gptb_tzgemm_static_scratch(dA, dB, got, tile_start, tile_end)
    torch.cuda.synchronize()
    assert ta.allocation_calls() == calls
    assert torch.cuda.mem_get_info()[0] == free_bytes
    assert torch.cuda.memory_allocated() == before
    return host(want), host(got)


def test_static_scratch_entry_matches_the_allocating_one_on_calls_in_a_row():
    setup()
    # reductions shared by 8, then 2 workgroups (the second call is smaller and finds the first
    # call's partial tiles and counters in the array), then a shape that needs no workspace,
    # then a tile range of a shared-reduction shape, then the largest workspace there is
    for M, N, K, rng_ in [(256, 512, 4608, None), (128, 128, 1024, None), (256, 256, 256, None),
                          (256, 512, 4608, (5, 23)), (128, 8192, 1024, None)]:
        assert (ta.tzgemm_parts(M, N, K) > 1) == (K >= 1024)
        want, got = both(M, N, K, seed=M + N + K, tile_start=rng_[0] if rng_ else 0,
                         tile_end=rng_[1] if rng_ else None)
        assert np.array_equal(want, got), (M, N, K)
        assert (want != -7.0).any()
    assert ta.spin_fail_flag() == 0


def test_the_allocating_entry_point_is_seen_by_the_allocation_count():
    """the witness itself: tacker_gptb_tzgemm on a fresh output buffer of a shared-reduction shape binds
    a workspace (one tkMalloc), so the count the test above relies on does move when something allocates"""
    setup()
    A, B = gemm_inputs(256, 512, 4608, 3)
    dA, dB = dev(A), dev(B)
    fresh = torch.zeros((256, 512), device="cuda:0")
    # torch hands out addresses again, and a binding nobody uses stays for the next kernel object on
    # the same output buffer: drop them all, so that this call has to bind (and allocate) one
    torch.cuda.synchronize()
    assert ta.lib().tacker_tzgemm_release_workspaces() == 0
    mallocs = ta.allocation_calls()[0]
    ta.gptb_tzgemm(dA, dB, fresh)
    torch.cuda.synchronize()
    assert ta.allocation_calls()[0] > mallocs


def test_static_scratch_entry_recorded_into_a_graph_and_replayed():
    """the call between tkStreamBeginCapture and tkStreamEndCapture runs nothing and allocates nothing;
    the graph replayed twice, with an eager call of a smaller shape on the same array in between, gives
    tacker_gptb_tzgemm's bits every time"""
    setup()
    l = ta.lib()
    M, N, K = 256, 512, 4608
    A, B = gemm_inputs(M, N, K, 11)
    dA, dB = dev(A), dev(B)
    want = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dA, dB, want)
    a2, b2 = gemm_inputs(128, 128, 1024, 12)
    dA2, dB2 = dev(a2), dev(b2)
    want2 = torch.zeros((128, 128), device="cuda:0")
    ta.gptb_tzgemm(dA2, dB2, want2)
    got = torch.full((M, N), -7.0, device="cuda:0")
    got2 = torch.full((128, 128), -7.0, device="cuda:0")
    torch.cuda.synchronize()
    stream = C.c_void_p()
    assert l.tkStreamCreate(C.byref(stream)) == 0
    try:
        calls = ta.allocation_calls()
        assert l.tkStreamBeginCapture(stream) == 0
        rc = l.tacker_gptb_tzgemm_static_scratch(dA.data_ptr(), dB.data_ptr(), got.data_ptr(), M, N, K, 0,
                                                 (M // 64) * (N // 64), 0, stream)
        graph = C.c_void_p()
        assert l.tkStreamEndCapture(stream, C.byref(graph)) == 0
        assert rc == 0
        assert ta.allocation_calls() == calls
        assert l.tkStreamSynchronize(stream) == 0
        assert (host(got) == -7.0).all()          # recorded, not run
        for replay in range(3):
            got.fill_(-7.0)
            torch.cuda.synchronize()
            assert l.tkGraphLaunch(graph, stream) == 0
            assert l.tkStreamSynchronize(stream) == 0
            assert np.array_equal(host(got), host(want)), replay
            # an eager, smaller call on the same array between the replays
            got2.fill_(-7.0)
            ta.gptb_tzgemm_static_scratch(dA2, dB2, got2)
            torch.cuda.synchronize()
            assert np.array_equal(host(got2), host(want2)), replay
        assert l.tkGraphExecDestroy(graph) == 0
    finally:
        l.tkStreamSynchronize(stream)
        l.tkStreamDestroy(stream)
    assert ta.spin_fail_flag() == 0


def test_static_scratch_entry_refuses_what_it_cannot_serve():
    setup()
    A, B = gemm_inputs(128, 128, 128)
    dA, dB = dev(A), dev(B)
    Cm = torch.zeros((128, 128), device="cuda:0")
    lib = ta.lib()
    s = torch.cuda.current_stream().cuda_stream
    assert lib.tacker_gptb_tzgemm_static_scratch(dA.data_ptr(), dB.data_ptr(), Cm.data_ptr(), 128, 128, 100, 0, 4, 0, s) == 3
    assert lib.tacker_gptb_tzgemm_static_scratch(dA.data_ptr(), dB.data_ptr(), Cm.data_ptr(), 128, 128, 128, 0, 5, 0, s) == 1
    assert lib.tacker_gptb_tzgemm_static_scratch(None, dB.data_ptr(), Cm.data_ptr(), 128, 128, 128, 0, 4, 0, s) == 1
    assert ta.tzgemm_workspace_bytes(128, 8192, 1024) <= (8 << 20) + (64 << 10)
