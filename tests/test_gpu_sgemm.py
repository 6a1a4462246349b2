"""GPU parity of the SGEMM partner (src/ori_kernel/sgemm_kernel.cu, src/gptb_kernel/sgemm_kernel.cu,
src/mix_kernel/tzgemm_sgemm.cu): bit-exact against the oracle's ordered evaluation (k ascending, one
fused multiply-add per step), in the natural launch, the GPTB form over any tiling of its
(blocks) x (k parts) position grid, fused with tzgemm in every variant, and as Creator builds it."""
import numpy as np
import pytest
import torch

import oracle
import tacker_amd as ta
from gpu_util import dev, gemm_inputs, gemm_tolerance_ok, host, setup

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    setup()


def inputs(M, N, K, seed=3):
    rng = np.random.default_rng(seed)
    A = rng.uniform(0, 1, (K, M)).astype(np.float32)
    B = rng.uniform(0, 1, (K, N)).astype(np.float32)
    C0 = rng.uniform(-1, 1, (N, M)).astype(np.float32)
    return A, B, C0


def bits(t):
    return host(t).view(np.uint32)


@pytest.mark.parametrize("M,N,K", [(128, 16, 8), (256, 48, 300), (384, 32, 1030), (128, 64, 3)])
def test_ori_and_gptb_forms_match_the_oracle_bit_for_bit(M, N, K):
    A, B, C0 = inputs(M, N, K, seed=M + K)
    want = oracle.sgemm(A, B, C0)
    dA, dB = dev(A), dev(B)
    c_ori, c_gptb, c_small = dev(C0), dev(C0), dev(C0)
    ta.ori_sgemm(dA, dB, c_ori)
    ta.gptb_sgemm(dA, dB, c_gptb)
    ta.gptb_sgemm(dA, dB, c_small, launch_grid=3, launch_block=128)
    for got in (c_ori, c_gptb, c_small):
        assert np.array_equal(bits(got), want.view(np.uint32))
    assert ta.sgemm_blocks(M, N, K) == oracle.sgemm_positions(M, N, K)
    assert ta.spin_fail_flag() == 0


@pytest.mark.parametrize("seed", range(8))
def test_any_ascending_tiling_of_the_position_grid_gives_the_one_kernel(seed):
    rng = np.random.default_rng(500 + seed)
    M, N, K = [(256, 48, 700), (128, 32, 1300), (384, 16, 520), (256, 64, 256)][seed % 4]
    A, B, C0 = inputs(M, N, K, seed=seed)
    want = oracle.sgemm(A, B, C0)
    total = ta.sgemm_blocks(M, N, K)
    cuts = sorted(set(rng.integers(0, total + 1, 4).tolist()) | {0, total})
    dA, dB, dC = dev(A), dev(B), dev(C0)
    out, W = C0.copy(), np.zeros((N, M), np.float32)
    for a, b in zip(cuts, cuts[1:]):
        grid = int(rng.choice([1, 7, 64, 256]))
        block = int(rng.choice([128, 256]))
        ta.gptb_sgemm(dA, dB, dC, start=a, end=b, launch_grid=grid, launch_block=block)
        out = oracle.sgemm(A, B, out, start=a, end=b, parts="chunks", W=W)
        # after every launch C is what the oracle has: untouched blocks old, finished blocks final
        assert np.array_equal(bits(dC), out.view(np.uint32)), (cuts, a, b, grid, block)
    assert np.array_equal(bits(dC), want.view(np.uint32))
    assert ta.spin_fail_flag() == 0


@pytest.mark.parametrize("variant", [None, "wave_128", "wave_256", "wave_384", "wave_512", "wg_1_1", "wg_1_2"])
def test_mix_tzgemm_sgemm(variant):
    M, N, K = 256, 256, 256
    A, B = gemm_inputs(M, N, K, seed=11)
    sA, sB, sC0 = inputs(256, 48, 700, seed=12)
    solo_c = torch.zeros((M, N), device="cuda:0")
    ta.gptb_tzgemm(dev(A), dev(B), solo_c)
    mix_c = torch.zeros((M, N), device="cuda:0")
    sC = dev(sC0)
    ta.mix_tzgemm_sgemm(dev(sA), dev(sB), sC, dev(A), dev(B), mix_c, variant=variant)
    assert np.array_equal(host(mix_c), host(solo_c))
    assert np.array_equal(bits(sC), oracle.sgemm(sA, sB, sC0).view(np.uint32))
    ok, fro, dmax = gemm_tolerance_ok(host(mix_c), oracle.tzgemm(A, B, f64=True), K)
    assert ok and fro <= 1e-5
    # a slice of the positions rides with a slice of the tiles; the rest follows in a second fused launch
    total = ta.sgemm_blocks(256, 48, 700)
    sC = dev(sC0)
    mix_c.zero_()
    ta.mix_tzgemm_sgemm(dev(sA), dev(sB), sC, dev(A), dev(B), mix_c, be_start=0, be_end=7, tile_start=0, tile_end=5,
                        variant=variant)
    ta.mix_tzgemm_sgemm(dev(sA), dev(sB), sC, dev(A), dev(B), mix_c, be_start=7, be_end=total, tile_start=5, tile_end=16,
                        variant=variant)
    assert np.array_equal(bits(sC), oracle.sgemm(sA, sB, sC0).view(np.uint32))
    assert np.array_equal(host(mix_c), host(solo_c))
    assert ta.spin_fail_flag() == 0


def test_partial_results_need_the_workspace_bound_to_c():
    # a hand-made launch of the GPTB kernel with k parts on a C the library never saw: nothing is computed
    # and the failure word says why
    import ctypes as C
    from gpu_util import launch
    M, N, K = 128, 16, 600
    A, B, C0 = inputs(M, N, K, seed=9)
    dA, dB = dev(A), dev(B)
    stray = dev(C0)
    i, p = C.c_int, lambda t: C.c_void_p(t.data_ptr())
    launch("gptb_sgemm", 4, 128, [p(dA), p(dB), p(stray), i(M), i(N), i(K), i(1), i(1), i(3), i(16), i(8), i(1),
                                  i(0), i(4), i(3), i(0)])
    torch.cuda.synchronize()
    assert np.array_equal(host(stray), C0)
    assert ta.spin_fail_flag() == 2 and ta.spin_fail_flag() == 0
    # with one part per block (the reference's kernel) no workspace is needed
    launch("gptb_sgemm", 4, 128, [p(dA), p(dB), p(stray), i(M), i(N), i(K), i(1), i(1), i(1), i(16), i(8), i(1),
                                  i(0), i(4), i(1), i(0)])
    torch.cuda.synchronize()
    assert np.array_equal(bits(stray), oracle.sgemm(A, B, C0).view(np.uint32))
    assert ta.spin_fail_flag() == 0


def test_creator_object_at_the_reference_size_matches_the_oracle_on_sampled_blocks():
    # createKernel("sgemm"): 4096 x 4128 x 4064, A and B uniform [0,1) from the library's seeded generator, C = 0
    # (src/ori_kernel/sgemm_kernel.cu:86-112); 528384 positions
    k = ta.create_kernel("sgemm")
    info = k.info()
    M, N, K = k.param(3, "int"), k.param(4, "int"), k.param(5, "int")
    assert (M, N, K) == (4096, 4128, 4064)
    assert (info["ptb_start"], info["ptb_end"]) == (0, 32 * 258 * 64) and (info["ori_grid_x"], info["ori_grid_y"]) == (32, 258)
    assert ta.lib().tkMemset(k.param(2), 0, M * N * 4) == 0          # the object is memoised: start from C = 0
    k.execute()
    torch.cuda.synchronize()
    A = ta.device_to_host(k.param(0), (K, M), np.float32)
    B = ta.device_to_host(k.param(1), (K, N), np.float32)
    got = ta.device_to_host(k.param(2), (N, M), np.float32)
    assert 0.0 <= A.min() and A.max() < 1.0 and abs(A.mean() - 0.5) < 1e-3
    zero = np.zeros((N, M), np.float32)
    for blk in (0, 4127, 8255):                                      # first, a middle and the last block
        bx, by = blk % 32, blk // 32
        want = oracle.sgemm(A, B, zero, start=blk, end=blk + 1)
        rows, cols = slice(bx * 128, bx * 128 + 128), slice(by * 16, by * 16 + 16)
        assert np.array_equal(got[cols, rows].view(np.uint32), want[cols, rows].view(np.uint32)), blk
    assert np.count_nonzero(got) == got.size
    assert ta.spin_fail_flag() == 0


def test_an_output_address_sgemm_has_used_serves_a_shared_reduction_tzgemm_afterwards():
    # sgemm leaves partial sums in the workspace bound to its C; tzgemm's shared reduction counts
    # arrivals there and needs them zero: the binding is cleared when the kind of kernel changes
    M, N, K = 256, 512, 4608
    assert ta.tzgemm_parts(M, N, K) > 1
    buf = torch.zeros(M * N, device="cuda:0")
    A, B, C0 = inputs(256, 512, 600, seed=9)
    c_s = buf.view(512, 256)
    c_s.copy_(dev(C0))
    ta.gptb_sgemm(dev(A), dev(B), c_s)
    assert np.array_equal(bits(c_s), oracle.sgemm(A, B, C0).view(np.uint32))
    gA, gB = gemm_inputs(M, N, K, 77)
    dA, dB = dev(gA), dev(gB)
    c_t = buf.view(M, N)
    assert c_t.data_ptr() == c_s.data_ptr()
    c_t.fill_(-7.0)
    other = torch.full((M, N), -7.0, device="cuda:0")
    ta.gptb_tzgemm(dA, dB, other)
    ta.gptb_tzgemm(dA, dB, c_t)
    assert np.array_equal(host(c_t), host(other))
    assert (host(c_t) != -7.0).all()
    # and back: sgemm on the address tzgemm has used
    c_s.copy_(dev(C0))
    ta.gptb_sgemm(dev(A), dev(B), c_s)
    assert np.array_equal(bits(c_s), oracle.sgemm(A, B, C0).view(np.uint32))
    assert ta.spin_fail_flag() == 0


def test_kernel_objects_of_both_kinds_on_one_output_address_in_any_launch_order():
    # a tzgemm object built on C, an sgemm object built on the same C afterwards, then launches in the
    # order sgemm (a range that ends inside the reduction: running sums stay in its workspace), the
    # older tzgemm object (its arrival counters must still be zero), the rest of sgemm (its sums must
    # still be there): each kernel has a workspace of its own under the one address
    M, N, K = 256, 512, 4608
    assert ta.tzgemm_parts(M, N, K) > 1
    buf = torch.zeros(M * N, device="cuda:0")
    gA, gB = gemm_inputs(M, N, K, 78)
    dA, dB = dev(gA), dev(gB)
    c_t = buf.view(M, N)
    tz = ta.gptb_create(ta.ori_tzgemm_create(dA, dB, c_t), 0, 0, 0, (M // 64) * (N // 64))
    A, B, C0 = inputs(256, 512, 600, seed=10)
    sA, sB = dev(A), dev(B)
    c_s = buf.view(512, 256)
    assert c_t.data_ptr() == c_s.data_ptr()
    positions = ta.sgemm_blocks(256, 512, 600)
    sg = ta.gptb_create(ta.ori_sgemm_create(sA, sB, c_s), 0, 0, 0, positions)
    other = torch.full((M, N), -7.0, device="cuda:0")
    ta.gptb_tzgemm(dA, dB, other)
    want_s = oracle.sgemm(A, B, C0).view(np.uint32)
    cut = positions // 2 + 3
    stash = torch.empty_like(c_s)
    for _ in range(2):                       # twice: whatever a round leaves behind serves the next
        c_s.copy_(dev(C0))
        sg.set_range(0, cut)
        sg.execute()
        stash.copy_(c_s)                     # sgemm's C so far (the tiles its range has finished)
        c_t.fill_(-7.0)
        tz.execute()
        assert np.array_equal(host(c_t), host(other))
        c_s.copy_(stash)
        sg.set_range(cut, positions)
        sg.execute()
        assert np.array_equal(bits(c_s), want_s)
    assert ta.spin_fail_flag() == 0
    sg.close()
    tz.close()
