"""GPU test of the tzgemm entry point that allocates nothing (its workspace is a static device
array of the library): output against tacker_gptb_tzgemm's, bit for bit, on calls in a row that
share the array, the later ones with smaller inputs."""
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
    before = torch.cuda.memory_allocated()
    ta.gptb_tzgemm_static_scratch(dA, dB, got, tile_start, tile_end)
    torch.cuda.synchronize()
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
