"""GPU tests of the conv->GEMM helpers, the VGG16 latency-critical task and the
TaskManager on the real device."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
import tacker_amd as ta
from gpu_util import dev, host, setup

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    setup()


@pytest.mark.parametrize("pad,stride,dil", [((1, 1), (1, 1), (1, 1)), ((0, 1), (2, 1), (1, 1)), ((2, 2), (1, 2), (2, 1))])
def test_im2col_bit_exact(pad, stride, dil):
    rng = np.random.default_rng(12)
    im = rng.uniform(-1, 1, (5, 17, 19)).astype(np.float32)
    want = oracle.im2col(im, (3, 3), pad, stride, dil)
    col = torch.zeros(want.shape, device="cuda:0")
    ta.im2col(dev(im), (3, 3), pad, stride, dil, col)
    assert np.array_equal(host(col), want)


def test_convert_fp32_to_fp16_rounds_to_nearest_even():
    rng = np.random.default_rng(13)
    x = np.concatenate([rng.uniform(-2, 2, 5000), rng.uniform(-1e-5, 1e-5, 1000), [0.0, 65504.0, 1e-8]]).astype(np.float32)
    out = torch.zeros(x.size, dtype=torch.float16, device="cuda:0")
    ta.convert_fp32_to_fp16(out, dev(x))
    assert np.array_equal(host(out).view(np.uint16), x.astype(np.float16).view(np.uint16))


def conv_reference(x_hwc, w, bias, C, Cout):
    """relu(1.1 * conv3x3(f16(x), w) + bias) in float64; x [H][W][>=C], w f16 [Np][Kp], k = (kh*3+kw)*C + c."""
    H, W = x_hwc.shape[:2]
    xp = np.zeros((H + 2, W + 2, C))
    xp[1:-1, 1:-1] = x_hwc[:, :, :C].astype(np.float16).astype(np.float64)
    wk = w[:Cout, :9 * C].astype(np.float64).reshape(Cout, 3, 3, C)
    out = np.zeros((H, W, Cout))
    for kh in range(3):
        for kw in range(3):
            out += np.einsum("hwc,nc->hwn", xp[kh:kh + H, kw:kw + W], wk[:, kh, kw])
    return np.maximum(float(np.float32(1.1)) * out + bias[:Cout].astype(np.float64), 0.0)


def read_act(task, idx):
    ptr, (H, W, C, ld) = task.activation(idx)
    return ta.device_to_host(ptr, (H, W, ld), np.float32), C


def test_vgg16_layers_match_direct_convolution():
    task = ta.LcTask("vgg16", 32, 64)
    task.execute()
    torch.cuda.synchronize()
    x = task.host_input().reshape(32, 64, 3)
    prev, prevC = x, 3
    for idx in range(4):                      # conv1_1, conv1_2, [pool], conv2_1, conv2_2
        w, b = task.conv_params(idx)
        got, Cout = read_act(task, idx)
        # the buffer holds the raw GEMM output; the layer that reads it adds the bias and rectifies
        got = np.maximum(got + b[None, None, :got.shape[2]], np.float32(0))
        if idx == 2:                          # a 2x2 max pool sits between conv1_2 and conv2_1
            H, W = prev.shape[:2]
            prev = prev.reshape(H // 2, 2, W // 2, 2, -1).max(axis=(1, 3))
        want = conv_reference(prev, w, b, prevC, Cout)
        np.testing.assert_allclose(got[:, :, :Cout], want, rtol=2e-4, atol=2e-4)
        assert np.all(got[:, :, Cout:] == 0)  # padded channels stay zero
        prev, prevC = got, Cout
    # kernel list as the scheduler sees it
    ks = task.kernels()
    assert [k["mixable"] for k in ks].count(2) == 13 and [k["mixable"] for k in ks].count(1) == 3
    task.close()


def test_vgg16_whole_forward_pass_matches_a_float64_model_of_it():
    # the whole network from the image to the logits in float64, never looking at the device's
    # intermediate results: operands rounded to f16 where the layers round them, 13 convolutions with
    # bias + ReLU, the five 2x2 max poolings, NHWC flattening, three fully connected layers
    task = ta.LcTask("vgg16", 32, 64)
    task.execute()
    torch.cuda.synchronize()
    f16 = lambda a: a.astype(np.float16).astype(np.float64)
    scale = float(np.float32(1.1))
    x = task.host_input().reshape(32, 64, 3).astype(np.float64)
    pool_before = {2, 4, 7, 10}               # convolutions whose input went through a pooling
    C = 3
    worst = 0.0
    for idx in range(13):
        w, b = task.conv_params(idx)
        if idx in pool_before:
            H, W = x.shape[:2]
            x = x.reshape(H // 2, 2, W // 2, 2, -1).max(axis=(1, 3))
        ptr, (H, W, Cout, ld) = task.activation(idx)
        assert x.shape == (H, W, C)
        want = conv_reference(x, w, b, C, Cout)
        raw = ta.device_to_host(ptr, (H, W, ld), np.float32)
        got = np.maximum(raw[:, :, :Cout] + b[None, None, :Cout], np.float32(0))
        tol = 1e-3 * np.abs(want).max()
        worst = max(worst, np.abs(got - want).max() / np.abs(want).max())
        assert np.abs(got - want).max() <= tol, (idx, np.abs(got - want).max(), tol)
        x, C = want, Cout
    H, W = x.shape[:2]
    v = x.reshape(H // 2, 2, W // 2, 2, -1).max(axis=(1, 3)).reshape(-1)      # pool5, NHWC flattening
    for idx in (13, 14, 15):
        w, b = task.conv_params(idx)
        ptr, (_, _, n_out, ld) = task.activation(idx)
        assert w.shape[1] >= v.size
        raw = scale * (w[:n_out, :v.size].astype(np.float64) @ f16(v))
        got_raw = ta.device_to_host(ptr, (ld,), np.float32)[:n_out]
        tol = 1e-3 * np.abs(raw).max()
        assert np.abs(got_raw - raw).max() <= tol, (idx, np.abs(got_raw - raw).max(), tol)
        worst = max(worst, np.abs(got_raw - raw).max() / np.abs(raw).max())
        v = np.maximum(raw + b[:n_out], 0.0)
    p, stride, n = task.logits()
    logits = ta.device_to_host(p, (n, stride), np.float32)[:, 0]
    assert n == raw.size and np.abs(logits - raw).max() <= 1e-3 * np.abs(raw).max()
    assert int(np.argmax(logits)) == int(np.argmax(raw)) or np.sort(raw)[-1] - np.sort(raw)[-2] < 2e-3 * np.abs(raw).max()
    assert np.abs(raw).max() > 0 and worst < 1e-3
    task.close()


@pytest.mark.parametrize("H,W,C,cs,pool", [(5, 7, 8, 8, 0), (8, 8, 64, 128, 0), (14, 14, 24, 32, 0), (3, 3, 16, 16, 0),
                                           (1, 1, 8, 8, 0), (2, 9, 40, 44, 0), (4, 6, 16, 128, 1), (7, 7, 64, 64, 1),
                                           (1, 2, 8, 12, 1)])
def test_scattered_conv_operand_equals_the_gathered_one(H, W, C, cs, pool):
    # A[m][(kh*3+kw)*C + c] built by scattering each pixel to the rows whose window covers it must be,
    # bit for bit, what the gather form builds -- including the zeros of border taps and of the columns
    # past 9*C, in a buffer that held something else before; with pool, what pooling first and gathering
    # from the pooled activations gives
    import ctypes as C_
    from gpu_util import launch
    rng = np.random.default_rng(H * 100 + W * 10 + C + pool)
    Hin, Win = (2 * H, 2 * W) if pool else (H, W)
    act = rng.uniform(-1, 1, (Hin, Win, cs)).astype(np.float32)
    bias = rng.uniform(-0.5, 0.5, cs).astype(np.float32)
    Kp = -(-9 * C // 128) * 128
    rows = H * W
    d_act, d_bias = dev(act), dev(bias)
    ptr = lambda t: C_.c_void_p(t.data_ptr())
    i = C_.c_int
    gathered = torch.zeros((rows, Kp), dtype=torch.float16, device="cuda:0")
    if pool:
        pooled = torch.zeros((H, W, cs), dtype=torch.float32, device="cuda:0")
        launch("maxpool2x2_nhwc", 64, 256, [ptr(d_act), i(Hin), i(Win), i(cs), ptr(pooled), ptr(d_bias), i(1)])
        launch("im2col_nhwc_f16", 64, 256, [ptr(pooled), i(H), i(W), i(C), i(cs), i(3), i(3), i(1), i(1), i(H), i(W),
                                            ptr(gathered), i(Kp), C_.c_void_p(0), i(1), i(0)])
    else:
        launch("im2col_nhwc_f16", 64, 256, [ptr(d_act), i(H), i(W), i(C), i(cs), i(3), i(3), i(1), i(1), i(H), i(W),
                                            ptr(gathered), i(Kp), ptr(d_bias), i(1), i(0)])
    scattered = torch.full((rows, Kp), 777.0, dtype=torch.float16, device="cuda:0")
    launch("im2col3x3_scatter_nhwc_f16", 64, 256, [ptr(d_act), i(H), i(W), i(C), i(cs), ptr(scattered), i(Kp),
                                                   ptr(d_bias), i(1), i(pool)])
    torch.cuda.synchronize()
    g = gathered.cpu().numpy().view(np.uint16)
    s_ = scattered.cpu().numpy().view(np.uint16)
    assert np.array_equal(g, s_)
    assert np.any(g[:, :9 * C] != 0) and np.all(g[:, 9 * C:] == 0)


@pytest.mark.parametrize("H,W,C,cs", [(9, 11, 3, 3), (6, 5, 3, 4), (4, 4, 5, 8)])
def test_gathered_operand_with_only_its_data_columns_rewritten(H, W, C, cs):
    # the first layer's operand: a buffer of its own whose columns past the data were zeroed once; a
    # gather that rewrites only columns [0, roundup8(9*C)) leaves what a gather of every column leaves,
    # which for every element is the plain definition A[m][(kh*3+kw)*C + c] = act[h+kh-1][w+kw-1][c]
    import ctypes as C_
    from gpu_util import launch
    rng = np.random.default_rng(H * W + C)
    act = rng.uniform(-1, 1, (H, W, cs)).astype(np.float32)
    d_act = dev(act)
    Kp, Kw = 128, (9 * C + 7) // 8 * 8
    ptr = lambda t: C_.c_void_p(t.data_ptr())
    i = C_.c_int
    outs = []
    for kw_arg, fill in ((0, 777.0), (Kw, 0.0)):
        A = torch.full((H * W, Kp), fill, dtype=torch.float16, device="cuda:0")
        launch("im2col_nhwc_f16", 64, 256, [ptr(d_act), i(H), i(W), i(C), i(cs), i(3), i(3), i(1), i(1), i(H), i(W),
                                            ptr(A), i(Kp), C_.c_void_p(0), i(0), i(kw_arg)])
        torch.cuda.synchronize()
        outs.append(A.cpu().numpy())
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16))
    padded = np.zeros((H + 2, W + 2, C), np.float32)
    padded[1:-1, 1:-1] = act[:, :, :C]
    want = np.zeros((H * W, Kp), np.float16)
    for kh in range(3):
        for kw in range(3):
            want[:, (kh * 3 + kw) * C:(kh * 3 + kw + 1) * C] = padded[kh:kh + H, kw:kw + W].reshape(H * W, C).astype(np.float16)
    assert np.array_equal(outs[0].view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("H,W,C,ld", [(14, 14, 512, 512), (4, 6, 24, 32), (2, 2, 8, 8)])
def test_pooled_classifier_input_equals_pooling_then_packing(H, W, C, ld):
    import ctypes as C_
    from gpu_util import launch
    rng = np.random.default_rng(H + W + C)
    raw = dev(rng.uniform(-1, 1, (H, W, ld)).astype(np.float32))
    bias = dev(rng.uniform(-0.5, 0.5, ld).astype(np.float32))
    n = (H // 2) * (W // 2) * C
    ptr = lambda t: C_.c_void_p(t.data_ptr())
    i = C_.c_int
    pooled = torch.zeros((H // 2, W // 2, ld), dtype=torch.float32, device="cuda:0")
    launch("maxpool2x2_nhwc", 64, 256, [ptr(raw), i(H), i(W), i(ld), ptr(pooled), ptr(bias), i(1)])
    want = torch.zeros(n, dtype=torch.float16, device="cuda:0")
    if ld == C:      # the packing kernel walks a dense vector: the pooled map flattens to one when ld == C
        launch("pack_fc_input", (n + 255) // 256, 256, [ptr(pooled), C_.c_long(1), C_.c_void_p(0), i(0), i(n), ptr(want)])
        want_bits = want.cpu().numpy().view(np.uint16)
    else:
        want_bits = pooled.cpu().numpy()[:, :, :C].reshape(-1).astype(np.float16).view(np.uint16)
    got = torch.full((n,), 777.0, dtype=torch.float16, device="cuda:0")
    launch("pack_fc_input_pooled", (n + 255) // 256, 256, [ptr(raw), i(W), i(ld), i(C), ptr(bias), i(1), i(n), ptr(got)])
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy().view(np.uint16), want_bits)
    assert np.any(want_bits != 0)
    # a grid smaller than the vector (the launcher caps it at a multiple of the CU count): same result
    for key, args in (("pack_fc_input_pooled", [ptr(raw), i(W), i(ld), i(C), ptr(bias), i(1), i(n)]),
                      ("pack_fc_input", [ptr(pooled), C_.c_long(1), C_.c_void_p(0), i(0), i(n)] if ld == C else None)):
        if args is None:
            continue
        few = torch.full((n,), 777.0, dtype=torch.float16, device="cuda:0")
        launch(key, 1, 64, args + [ptr(few)])
        torch.cuda.synchronize()
        assert np.array_equal(few.cpu().numpy().view(np.uint16), want_bits), key


def test_task_manager_colocation_keeps_lc_results_and_reports():
    task = ta.LcTask("vgg16", 64, 64)
    task.execute()
    torch.cuda.synchronize()
    p, stride, n = task.logits()
    solo_logits = ta.device_to_host(p, (n, stride), np.float32)[:, 0].copy()
    assert np.isfinite(solo_logits).all() and np.abs(solo_logits).max() > 0

    tm = ta.TaskManager(task, "stencil", "lbm")
    tm.configure(qos_budget_ms=50.0, guard_ms=0.5, warmup=1, profile=3, queries=4, verbose=0)
    rep = tm.run("aker", second_stage=True)
    torch.cuda.synchronize()
    mixed_logits = ta.device_to_host(p, (n, stride), np.float32)[:, 0]
    assert np.array_equal(mixed_logits, solo_logits)      # fused launches leave the LC numerics untouched
    assert rep["mixable_times"] == 16 and rep["lc_solo_ms"] > 0 and rep["be1_solo_ms"] > 0
    assert rep["n_colocated"] == 4 and rep["n_solo"] == 3
    lat = tm.latencies()
    assert len(lat) == 4 and all(0 < v < 50.0 for v in lat)
    assert rep["qos_headroom_left_ms"] > 0
    assert tm.latencies(kind="e2e_solo") == []
    # whole queries between one pair of events: same logits, and never longer than the sum of
    # per-kernel intervals with a synchronisation after each kernel
    tm.set_end_to_end(5)
    tm.run("aker", second_stage=False)
    torch.cuda.synchronize()
    assert np.array_equal(ta.device_to_host(p, (n, stride), np.float32)[:, 0], solo_logits)
    for kind in ("e2e_solo", "e2e_colocated", "e2e_solo_wall", "e2e_colocated_wall"):
        got = tm.latencies(kind=kind)
        assert len(got) == 5 and all(0 < v < 50.0 for v in got), kind
    for kind in ("e2e_graph", "e2e_graph_wall"):
        got = tm.latencies(kind=kind)
        assert len(got) == 5 and all(0 < v < 50.0 for v in got), kind
    assert min(tm.latencies(kind="e2e_solo")) < min(tm.latencies(solo=True))
    assert all(w >= e - 1e-3 for w, e in zip(tm.latencies(kind="e2e_solo_wall"), tm.latencies(kind="e2e_solo")))
    tm.set_end_to_end(0)
    rep2 = tm.run("tacker", second_stage=False)
    assert rep2["n_colocated"] == 4
    torch.cuda.synchronize()
    assert np.array_equal(ta.device_to_host(p, (n, stride), np.float32)[:, 0], solo_logits)
    tm.close()
    task.close()


def test_mix_entry_points_on_the_global_operands_match_the_oracle():
    # mixcublasSgemm / mixcudnnConvolutionForward (src/TaskManager.cu:309-400, 125-306) for a latency-critical
    # kernel that brings no operands: the GEMM reads the library's seeded operand buffers
    from gpu_util import C0, C1, gemm_tolerance_ok, stencil_inputs
    A0 = stencil_inputs(6, 20, 200, seed=41)
    for call, dims in ((lambda g, a, b: ta.mix_cublas_sgemm([200, 100, 300], g, a, b), (200, 100, 300)),
                       (lambda g, a, b: ta.mix_cudnn_convolution_forward([1, 8, 20, 20, 32, 8, 3, 3, 1, 1, 1, 1, 1, 1],
                                                                         g, a, b), (400, 32, 72))):
        M, N, K, tiles = ta.tzgemm_grid_dim(*dims)
        a0 = dev(A0)
        out = a0.clone()
        ori = ta.ori_stencil_create(C0, C1, a0, out)
        blocks = ta.stencil_blocks(200, 20, 6)
        g = ta.gptb_create(ori, 0, 0, 0, blocks)
        call(g, 0, blocks)
        torch.cuda.synchronize()
        pa, pb, pc, _ = ta.global_gemm_buffers()
        A = ta.device_to_host(pa, (M, K), np.float16)
        B = ta.device_to_host(pb, (N, K), np.float16)
        got = ta.device_to_host(pc, (M, N), np.float32)
        assert np.abs(A.astype(np.float32)).max() > 0
        ok, fro, dmax = gemm_tolerance_ok(got, oracle.tzgemm(A, B, f64=True), K)
        assert ok and fro <= 1e-5, (dims, fro, dmax)
        assert np.array_equal(host(out).view(np.uint32), oracle.stencil(C0, C1, A0, A0).view(np.uint32)), dims
        # a partial range leaves the other positions of the sweep untouched; an empty one runs the GEMM alone
        out.copy_(a0)
        call(g, 1, 3)
        want = oracle.stencil_gptb(C0, C1, A0, A0, start=1, end=3, gdz="runs")
        assert np.array_equal(host(out).view(np.uint32), want.view(np.uint32)), dims
        out.copy_(a0)
        call(g, 2, 2)
        assert np.array_equal(host(out), A0)
    assert ta.spin_fail_flag() == 0


def test_task_manager_colocates_mrif_and_pairs_it_with_lbm():
    # the fifth best-effort kernel through the same scheduler: tzgemm_mrif launches in stage 1,
    # the lbm_mrif pair (src/mix_kernel/lbm_mrif_1_3.cu) in stage 2
    task = ta.LcTask("vgg16", 64, 64)
    task.execute()
    torch.cuda.synchronize()
    p, stride, n = task.logits()
    solo_logits = ta.device_to_host(p, (n, stride), np.float32)[:, 0].copy()
    tm = ta.TaskManager(task, "lbm", "mrif")
    tm.configure(qos_budget_ms=50.0, guard_ms=0.5, warmup=1, profile=3, queries=3, verbose=0)
    rep = tm.run("aker", second_stage=True)
    torch.cuda.synchronize()
    assert np.array_equal(ta.device_to_host(p, (n, stride), np.float32)[:, 0], solo_logits)
    assert rep["mixable_times"] == 16 and rep["be1_solo_ms"] > 0 and rep["n_colocated"] == 3
    tm.close()
    tm = ta.TaskManager(task, "mrif", None)
    tm.configure(qos_budget_ms=50.0, guard_ms=0.5, warmup=1, profile=3, queries=3, verbose=0)
    rep = tm.run("aker", second_stage=False)
    torch.cuda.synchronize()
    assert np.array_equal(ta.device_to_host(p, (n, stride), np.float32)[:, 0], solo_logits)
    assert rep["n_colocated"] == 3 and ta.spin_fail_flag() == 0
    tm.close()
    task.close()


def test_create_kernel_objects_run_and_match_oracle_for_cp():
    k = ta.create_kernel("cp")
    info = k.info()
    # 32 x 512 blocks of 128 x 8 points, each in 4 parts of its x points
    assert (info["ptb_start"], info["ptb_end"]) == (0, 65536) and info["ori_grid_x"] == 32 and info["ori_grid_y"] == 512
    assert info["nparams"] == 3 + 6 and k.param(0, "int") == 64 and k.param(1, "float") == np.float32(0.1)
    # the object is memoised and the kernel accumulates: start from the zeroed grid its constructor made
    assert ta.lib().tkMemset(k.param(2), 0, 4096 * 4096 * 4) == 0
    k.execute()
    torch.cuda.synchronize()
    # the object's own inputs (src/ori_kernel/cp_kernel.cu:66-100): atoms 1..64 of the seeded
    # 4000, plane z = 0, a zeroed 4096 x 4096 grid; rows of blocks from the top, middle and bottom
    grid = ta.device_to_host(k.param(2), (4096, 4096), np.float32)
    consts = oracle.cp_atoms_to_const(oracle.cp_initatoms(4000)[1:65], 0.0)
    for first_row in (0, 2048, 4088):
        rows = slice(first_row, first_row + 8)
        lo = (first_row // 8) * 32                    # the 32 blocks of this row of blocks
        want = oracle.cp(consts, np.zeros((4096, 4096), np.float32), start=lo, end=lo + 32)[rows]
        assert np.array_equal(grid[rows].view(np.uint32), want.view(np.uint32)), first_row
    assert np.count_nonzero(grid) == grid.size
    for name in ("stencil", "lbm", "mriq", "mrif"):
        ta.create_kernel(name).execute()
    torch.cuda.synchronize()
    assert ta.spin_fail_flag() == 0


def test_a_recorded_query_gives_the_eager_logits_on_every_replay():
    """The query's launches recorded once and launched as one graph: replayed several times, with the
    input staged again, eager queries, other kernels and synchronisations between the replays, and
    every replay's logits compared bit for bit with the eager query's."""
    task = ta.LcTask("vgg16", 64, 64)
    task.execute()
    torch.cuda.synchronize()
    p, stride, n = task.logits()
    want = ta.device_to_host(p, (n, stride), np.float32)[:, 0].copy()
    assert np.isfinite(want).all() and np.abs(want).max() > 0
    l = ta.lib()
    stream = C.c_void_p()
    assert l.tkStreamCreate(C.byref(stream)) == 0
    with pytest.raises(ta.TackerError, match="null stream"):
        task.capture(None)
    graph = task.capture(stream)
    x = torch.randn(1 << 20, device="cuda")
    for replay in range(6):
        # wipe the logits so that a replay that ran nothing cannot pass on the last one's result
        assert l.tkMemset(p, 0xFF, n * stride * 4) == 0
        torch.cuda.synchronize()
        task.stage_input()
        graph.launch(stream)
        assert l.tkStreamSynchronize(stream) == 0
        got = ta.device_to_host(p, (n, stride), np.float32)[:, 0]
        assert np.array_equal(got, want), replay
        # the program's own eager work between replays: another query kernel by kernel, a library reduction
        if replay % 2 == 0:
            task.execute()
        assert torch.isfinite(x.sum()).item()
        torch.cuda.synchronize()
    graph.close()
    assert l.tkStreamDestroy(stream) == 0
    task.close()
