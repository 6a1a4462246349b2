#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: the fused tzgemm + stencil launch
against serial launches of the same two kernels.

Workload (benchmark configuration 2): tzgemm fp16 2048x2048x2048 (uniform[-1,1], fp32
accumulate, alpha 1.1) + Parboil 7-point Jacobi stencil on an fp32 512x512x64 grid
(uniform[0,1], c0=1/6, c1=1/36), 100 iterations with pointer swap.  One "step" is
the whole 100-iteration job: serial = 100 x (1 GEMM launch + 1 sweep launch) on one
stream, fused = 100 fused launches (GEMM tiles [0,1024) + stencil blocks [0,1024)).

Prints ONE JSON line: value = serial time / fused time, with the roofline of the
fused kernel and the CPU baseline (the oracle restatement on the host cores).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12          # B/s, MI355X HBM3E
MFMA_F16_PEAK = 2.5e15     # flop/s, dense fp16 MFMA

# HBM-side bytes one fused launch moves, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this
# file scaled by what the same counters read for a 64 MiB copy (x1.9988 and x1.0000); the summary with
# the commands is profiles/pmc_hbm_traffic_bench_tzgemm2048_stencil512x512x64.txt
FUSED_HBM_TRAFFIC_BYTES = 2.044e8

GEMM_MNK = (2048, 2048, 2048)
STENCIL_DIMS = (64, 512, 512)      # nz, ny, nx
ITERATIONS = 100


def trimmed_mean(xs):
    xs = sorted(xs)
    if len(xs) >= 5:
        k = len(xs) // 4
        xs = xs[k:len(xs) - k]
    return sum(xs) / len(xs)


def cpu_baseline(A, B, A0, c0, c1):
    """The oracle (CPU port of the reference kernels) on the host cores: 3 GEMMs and
    30 sweeps timed (about 20 core-seconds), scaled to the job's 100 + 100."""
    import numpy as np
    import oracle
    gemms, sweeps = 3, 30
    t0 = time.perf_counter()
    for _ in range(gemms):
        oracle.tzgemm(A, B)
    t_gemm = (time.perf_counter() - t0) / gemms
    a, b = A0.copy(), A0.copy()
    t0 = time.perf_counter()
    for _ in range(sweeps):
        b = oracle.stencil(c0, c1, a, b)
        a, b = b, a
    t_sweep = (time.perf_counter() - t0) / sweeps
    ms = (t_gemm + t_sweep) * ITERATIONS * 1e3
    return {"value": round(ms, 1), "unit": "ms_per_step", "cores": oracle.num_threads(), "kind": "port",
            "sample": "oracle/tacker_oracle.c with OpenMP: %d tzgemm 2048^3 (%.2f s each) + %d stencil sweeps "
                      "512x512x64 (%.4f s each), scaled to 100 + 100" % (gemms, t_gemm, sweeps, t_sweep)}


def pair_leg(ta, torch, np, name, stream):
    """One of the other fused pairs (benchmark configurations 3 and 4): each kernel alone, serial, and the
    fused launch over the full ranges, 200 launches each, median of 3 rounds."""
    import statistics
    rng = np.random.default_rng(1337)

    def gemm(M, N, K):
        A = torch.from_numpy(rng.uniform(-1, 1, (M, K)).astype(np.float16)).cuda()
        B = torch.from_numpy(rng.uniform(-1, 1, (N, K)).astype(np.float16)).cuda()
        Cm = torch.zeros((M, N), device="cuda:0")
        tiles = (M // 64) * (N // 64)
        return ta.gptb_create(ta.ori_tzgemm_create(A, B, Cm), 0, 0, 0, tiles), tiles, 2.0 * M * N * K

    swap = None             # exchanges the best-effort kernel's input and output grid after a launch
    reset = None            # puts the best-effort kernel's output back to its start before a timed round
    n = 200                 # launches per timed round
    if name == "cp":        # Coulomb potential, 4096x4096 grid, 64 atoms (the Creator's instance, src/Creator.cu:23-37)
        volx = voly = 4096
        atoms = ta.cp_initatoms(4000, volx, voly, 1, 0.1)
        ta.cp_set_atoms(atoms[1:65], 0.0)
        grid = torch.zeros((voly, volx), device="cuda:0")
        be_ori = ta.ori_cp_create(64, 0.1, grid)
        nblk = ta.cp_blocks(volx, voly)
        tz, tiles, flop = gemm(2048, 2048, 2048)
        work = {"bound": "valu", "pairs": 64.0 * volx * voly}
        label = "tzgemm 2048^3 + cp 4096x4096, 64 atoms (reference mix tzgemm_cp; named by the north star)"
    elif name == "sgemm":   # Parboil SGEMM, 4096 x 4128 x 4064 (the Creator's instance, src/ori_kernel/sgemm_kernel.cu:86-88)
        sM, sN, sK = 4096, 4128, 4064
        sA = torch.rand((sK, sM), device="cuda:0")
        sB = torch.rand((sK, sN), device="cuda:0")
        sC = torch.zeros((sN, sM), device="cuda:0")
        be_ori = ta.ori_sgemm_create(sA, sB, sC)
        nblk = ta.sgemm_blocks(sM, sN, sK)
        tz, tiles, flop = gemm(2048, 2048, 2048)
        work = {"bound": "valu", "pairs": float(sM) * sN * sK}
        label = "tzgemm 2048^3 + sgemm 4096x4128x4064 fp32 (reference mix tzgemm_sgemm)"
        reset = sC.zero_        # C = 2 C + 2 A B doubles with every pass: start every timed round from zero
        n = 50
    elif name == "cutcp":   # cutoff Coulomb potential, the Creator's instance (src/ori_kernel/cutcp_kernel.cu:181-263)
        n_pts, count = 208, 70000
        atoms = np.empty((count, 4), np.float32)
        atoms[:, :3] = rng.uniform(0, (n_pts - 1) * 0.5, (count, 3))
        atoms[:, 3] = rng.uniform(0.1, 1, count) * rng.choice([-1, 1], count)
        inp = ta.CutcpInput(atoms, (0, 0, 0), n_pts, n_pts, n_pts, 0.5, 12.0, regions=(26, 26, 2))
        be_ori = ta.ori_cutcp_create(inp, 144.0, 0.006944)
        nblk = inp.blocks()
        tz, tiles, flop = gemm(2048, 2048, 2048)
        # atom-point pairs: 335 neighbour bins of each of the 1352 regions, their atoms, 512 points
        filled = float(np.count_nonzero(inp.host_bins[..., 3])) / inp.host_bins[..., 3].size * 8
        work = {"bound": "valu", "pairs": 26 * 26 * 2 * 512.0 * len(inp.nbr) * filled}
        label = "tzgemm 2048^3 + cutcp 208^3 lattice, 70000 atoms, 26x26x2 regions (reference mix tzgemm_cutcp)"
    elif name == "fft":     # Parboil FFT, 10240 transforms of 256 points (the Creator's instance, src/ori_kernel/fft_kernel.cu:87-115)
        batches = 10240
        source = torch.from_numpy(rng.uniform(-1, 1, (batches, 256, 2)).astype(np.float32)).cuda()
        data = source.clone()
        be_ori = ta.ori_fft_create(data)
        nblk = batches
        tz, tiles, flop = gemm(2048, 2048, 2048)
        work = {"bound": "hbm", "algorithmic_bytes": 2.0 * batches * 256 * 8}
        label = "tzgemm 2048^3 + fft 10240 x 256 points (reference mix tzgemm_fft)"
        reset = lambda: data.copy_(source)   # in place: every pass multiplies the magnitudes by 16
        n = 25
    elif name == "nn":      # Rodinia nn, 256 x 2560000 records (the Creator's instance, src/ori_kernel/nn_kernel.cu:46)
        records = 256 * 2560000
        loc = torch.rand((records, 2), device="cuda:0") * 90.0
        dist = torch.zeros(records, device="cuda:0")
        be_ori = ta.ori_nn_create(loc, dist, 30.0, 90.0)
        nblk = ta.nn_blocks(records)
        tz, tiles, flop = gemm(2048, 2048, 2048)
        work = {"bound": "hbm", "algorithmic_bytes": 12.0 * records}
        label = "tzgemm 2048^3 + nn 655360000 records (reference mix tzgemm_nn)"
        n = 10
    elif name == "hot3d":   # Rodinia hotspot3D, 16384 x 8192 x 8 cells (the Creator's instance, src/ori_kernel/hot3d_kernel.cu:80-82)
        nx, ny, nz = 16384, 8192, 8
        power = torch.rand((nz, ny, nx), device="cuda:0") * 0.01
        t_in = torch.rand((nz, ny, nx), device="cuda:0") * 20.0 + 320.0
        t_out = torch.zeros((nz, ny, nx), device="cuda:0")
        be_ori = ta.ori_hot3d_create(power, t_in, t_out)
        nblk = ta.hot3d_blocks(nx, ny)
        tz, tiles, flop = gemm(2048, 2048, 2048)
        work = {"bound": "hbm", "algorithmic_bytes": 12.0 * nx * ny * nz}
        label = "tzgemm 2048^3 + hotspot3D 16384x8192x8 (reference mix tzgemm_hot3d)"
        n = 6
    elif name == "lava":    # Rodinia lavaMD, 60^3 boxes of 100 particles (src/ori_kernel/lava_kernel.cu:163-175)
        boxes1d = 60
        particles = 100 * boxes1d ** 3
        rv = torch.rand((particles, 4), device="cuda:0") * 0.9 + 0.1
        qv = torch.rand(particles, device="cuda:0") * 0.9 + 0.1
        fv = torch.zeros((particles, 4), device="cuda:0")
        be_ori = ta.ori_lava_create(0.5, rv, qv, fv)
        nblk = ta.lava_blocks(boxes1d)
        tz, tiles, flop = gemm(2048, 2048, 2048)
        # particle pairs: every box against itself and its neighbours (58^3 inner boxes have 26, faces fewer)
        per_edge = [2 if c in (0, boxes1d - 1) else 3 for c in range(boxes1d)]
        box_pairs = float(sum(per_edge)) ** 3
        work = {"bound": "valu", "pairs": box_pairs * 100.0 * 100.0}
        label = "tzgemm 2048^3 + lavaMD 60^3 boxes x 100 particles (reference mix tzgemm_lava)"
        reset = fv.zero_        # the forces accumulate from launch to launch
        n = 3
    elif name == "path":    # Rodinia pathfinder, 1200 columns, pyramid of 125 rows (src/ori_kernel/path_kernel.cu:102)
        cols, height = 1200, 125
        wall = torch.from_numpy(rng.integers(0, 10, (height, cols), dtype=np.int32)).cuda()
        src_row = torch.from_numpy(rng.integers(0, 10, cols, dtype=np.int32)).cuda()
        result_row = torch.zeros(cols, dtype=torch.int32, device="cuda:0")
        be_ori = ta.ori_path_create(height, wall, src_row, result_row)
        nblk = ta.path_blocks(cols, height)
        tz, tiles, flop = gemm(2048, 2048, 2048)
        work = {"bound": "valu", "pairs": 256.0 * nblk * height}   # column updates of the 200 windows
        label = "tzgemm 2048^3 + pathfinder 1200 columns x 125 rows (reference mix tzgemm_path)"
    elif name == "lbm":     # D3Q19, 120x120x150, rest equilibrium + noise, 5 % obstacle cells
        sx, sy, sz = 120, 120, 150
        cells = sx * sy * sz
        w = np.array([1 / 3] + [1 / 18] * 6 + [1 / 36] * 12, np.float32)
        g = np.zeros((20, cells), np.float32)
        g[:19] = w[:, None] + rng.uniform(0, 1e-3, (19, cells)).astype(np.float32)
        g[19] = (rng.uniform(0, 1, cells) < 0.05).astype(np.uint32).view(np.float32)
        src = torch.from_numpy(g.reshape(-1)).cuda()
        dst = src.clone()
        be_ori = ta.ori_lbm_create(src, dst, sx, sy, sz)
        swap = be_ori.swap_buffers     # every launch is the next step of the simulation: src <-> dst
        nblk = sy * sz
        tz, tiles, flop = gemm(4096, 4096, 1024)
        work = {"bound": "hbm", "algorithmic_bytes": 156.0 * cells}
        label = "configs[2]: tzgemm 4096x4096x1024 + lbm 120x120x150 (one step per launch, src and dst exchanged after each)"
    elif name == "mrif":    # mri-fhd, numK 2048, numX 262144 (the reference's tzgemm_mrif mix; no benchmark configuration of its own)
        numK, numX = 2048, 262144
        k = rng.uniform(-0.5, 0.5, (numK, 3)).astype(np.float32)
        phi = rng.uniform(0, 1, (2, numK)).astype(np.float32)
        d = rng.uniform(0, 1, (2, numK)).astype(np.float32)
        rho = [torch.zeros(numK, device="cuda:0") for _ in range(2)]
        ta.mrif_rhophi(*[torch.from_numpy(a).cuda() for a in (phi[0], phi[1], d[0], d[1])], rho[0], rho[1])
        kv = np.concatenate([k, rho[0].cpu().numpy()[:, None], rho[1].cpu().numpy()[:, None]], 1).astype(np.float32)
        ta.mrif_set_kvalues(kv)
        xyz = [torch.from_numpy(rng.uniform(-0.5, 0.5, numX).astype(np.float32)).cuda() for _ in range(3)]
        outR, outI = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
        be_ori = ta.ori_mrif_create(numK, xyz[0], xyz[1], xyz[2], outR, outI)
        nblk = ta.mrif_blocks(numK, numX)
        tz, tiles, flop = gemm(2048, 2048, 2048)
        work = {"bound": "valu", "pairs": float(numK) * numX}
        label = "tzgemm 2048^3 + mri-fhd numK 2048, numX 262144 (reference mix tzgemm_mrif)"
    else:                   # mri-q, numK 2048, numX 262144
        numK, numX = 2048, 262144
        k = rng.uniform(-0.5, 0.5, (numK, 3)).astype(np.float32)
        phi = rng.uniform(0, 1, (2, numK)).astype(np.float32)
        kv = np.concatenate([k, (phi[0] * phi[0] + phi[1] * phi[1])[:, None]], 1).astype(np.float32)
        ta.mriq_set_kvalues(kv)
        xyz = [torch.from_numpy(rng.uniform(-0.5, 0.5, numX).astype(np.float32)).cuda() for _ in range(3)]
        Qr, Qi = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
        be_ori = ta.ori_mriq_create(numK, xyz[0], xyz[1], xyz[2], Qr, Qi)
        nblk = ta.mriq_blocks(numK, numX)
        tz, tiles, flop = gemm(2048, 2048, 2048)
        work = {"bound": "valu", "pairs": float(numK) * numX}
        label = "configs[3]: tzgemm 2048^3 + mri-q numK 2048, numX 262144"
    be = ta.gptb_create(be_ori, 0, 0, 0, nblk)
    mix = ta.mix_create(be, tz, 0, nblk, 0, tiles)
    # the slice TaskManager would co-locate with this GEMM: tiles x block_ratio(K) best-effort blocks
    gemm_k = 1024 if name == "lbm" else 2048
    ratio = ta.lib().tacker_qos_block_ratio(name.encode(), gemm_k)
    slice_blocks = min(int(tiles * ratio), nblk)
    be_slice = ta.gptb_create(be_ori, 0, 0, 0, max(slice_blocks, 1))
    mix_slice = ta.mix_create(be, tz, 0, slice_blocks, 0, tiles)
    e0, e1 = ta.Event(), ta.Event()

    def timed(fn):
        nonlocal n
        if reset:
            reset()
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(n):
            fn()
        e1.record(stream)
        e1.synchronize()
        return e0.elapsed_ms(e1) / n * 1e3

    def be_alone():
        be.execute(stream)
        if swap:
            swap()

    def serial():
        tz.execute(stream)
        be_alone()

    def fused():
        mix.execute(stream)
        if swap:
            swap()

    def serial_slice():
        tz.execute(stream)
        be_slice.execute(stream)

    cases = {"gemm_us": lambda: tz.execute(stream), "be_us": be_alone, "serial_us": serial, "fused_us": fused}
    if slice_blocks > 0:
        cases["slice_serial_us"] = serial_slice
        cases["slice_fused_us"] = lambda: mix_slice.execute(stream)
    rounds = {key: [] for key in cases}
    for _ in range(3):
        for key, fn in cases.items():
            rounds[key].append(timed(fn))
    out = {key: round(statistics.median(v), 2) for key, v in rounds.items()}
    out["workload"] = label
    out["speedup"] = round(out["serial_us"] / out["fused_us"], 4)
    out["slice_blocks"] = slice_blocks
    out["be_blocks"] = nblk
    if slice_blocks > 0:
        out["slice_speedup"] = round(out["slice_serial_us"] / out["slice_fused_us"], 4)
    # what TaskManager credits a co-located slice with: the GEMM alone plus the slice at the whole kernel's
    # rate (src/TaskManager.cu:626-640) -- the slice launched alone runs below that rate, which flatters
    # slice_speedup
    if slice_blocks > 0:
        out["slice_serial_at_kernel_rate_us"] = round(out["gemm_us"] + out["be_us"] * slice_blocks / nblk, 2)
        out["slice_speedup_at_kernel_rate"] = round(out["slice_serial_at_kernel_rate_us"] / out["slice_fused_us"], 4)
    if out["be_us"] > 1.3 * out["gemm_us"] and slice_blocks > 0:
        # The longer best-effort kernel spread over the GEMMs it rides with, the way the scheduler does it in
        # Aker mode: consecutive fused launches, each carrying the next slice_blocks block positions (a cursor),
        # against as many GEMM launches plus the best-effort kernel alone over the same positions.  At most 64
        # launches are timed (the first 64 slices of kernels that need more).
        n_cur = min(64, (nblk + slice_blocks - 1) // slice_blocks)
        bounds = [min(nblk, slice_blocks * i) for i in range(n_cur + 1)]
        mix_cur = ta.mix_create(be, tz, 0, 0, 0, tiles)
        be_part = be if bounds[-1] == nblk else ta.gptb_create(be_ori, 0, 0, 0, bounds[-1])

        def cursor_fused():
            for i in range(n_cur):
                mix_cur.set_range(bounds[i], bounds[i + 1], 0, tiles)
                mix_cur.execute(stream)

        def cursor_serial():
            for _ in range(n_cur):
                tz.execute(stream)
            be_part.execute(stream)

        n = 40 if n_cur <= 30 else 10
        cur = {"cursor_serial_us": [], "cursor_fused_us": []}
        for _ in range(3):
            cur["cursor_serial_us"].append(timed(cursor_serial))
            cur["cursor_fused_us"].append(timed(cursor_fused))
        out.update({key: round(statistics.median(v), 2) for key, v in cur.items()})
        out["cursor_launches"] = n_cur
        out["cursor_blocks"] = bounds[-1]
        out["cursor_speedup"] = round(out["cursor_serial_us"] / out["cursor_fused_us"], 4)
    # the scheduler's decisions for this pair (kinfo): Aker mode co-locates slice_blocks positions with a GEMM
    # of this K (0 = never fuses it at this K); Tacker mode lets the whole kernel ride only if kinfo's measured
    # whole-kernel gain says that it pays, and falls back to the Aker slice otherwise
    whole = ta.lib().tacker_qos_whole_kernel_gain(name.encode())
    out["scheduler"] = {"aker_slice_blocks": slice_blocks, "aker_fuses": bool(slice_blocks > 0),
                        "kinfo_whole_kernel_gain": round(whole, 4), "tacker_fuses_whole_kernel": bool(whole >= 1.03)}
    picked = []
    if slice_blocks > 0:
        picked.append(out.get("cursor_speedup", out["slice_speedup_at_kernel_rate"]))
    if whole >= 1.03:    # QosPolicy::kWholeKernelGainMin
        picked.append(out["speedup"])
    out["scheduler"]["slowest_form_it_would_pick"] = round(min(picked), 4) if picked else None
    out["gemm_tflops_alone"] = round(flop / out["gemm_us"] / 1e6, 1)
    if work["bound"] == "hbm":
        out["be_gbps_alone"] = round(work["algorithmic_bytes"] / out["be_us"] / 1e3, 1)
        out["be_frac_of_hbm_peak"] = round(work["algorithmic_bytes"] / (out["be_us"] * 1e-6) / HBM_PEAK, 4)
    else:
        out["be_gpairs_per_s_alone"] = round(work["pairs"] / out["be_us"] / 1e3, 1)
    return out


def gemm_leg(ta, torch, np, stream):
    """tzgemm alone at the shapes of the benchmark configurations and at 4096^3, with a yardstick from the same
    GPU beside each: torch.matmul on the same fp16 operands (the vendor library's kernel; time only)."""
    import statistics
    rng = np.random.default_rng(1337)
    out = {}
    for M, N, K in ((1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 1024), (4096, 4096, 4096)):
        A = torch.from_numpy(rng.uniform(-1, 1, (M, K)).astype(np.float16)).cuda()
        B = torch.from_numpy(rng.uniform(-1, 1, (N, K)).astype(np.float16)).cuda()
        Cm = torch.zeros((M, N), device="cuda:0")
        tz = ta.gptb_create(ta.ori_tzgemm_create(A, B, Cm), 0, 0, 0, (M // 64) * (N // 64))
        Bt = B.t()
        e0, e1 = ta.Event(), ta.Event()
        n = 50

        def timed(fn):
            # 20 ms of the same kernel first: the clocks of a GPU that has just been copying operands take
            # milliseconds to settle, and whichever kernel is timed first would pay for it
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < 0.02:
                for _ in range(10):
                    fn()
                torch.cuda.synchronize()
            e0.record(stream)
            for _ in range(n):
                fn()
            e1.record(stream)
            e1.synchronize()
            return e0.elapsed_ms(e1) / n * 1e3

        # the library with the output type tzgemm has (an fp32 C is twice the bytes of torch.matmul's fp16 C);
        # None where this torch build does not offer it
        candidates = {"ours": lambda: tz.execute(stream), "lib": lambda: torch.matmul(A, Bt)}
        try:
            torch.mm(A, Bt, out_dtype=torch.float32)
            candidates["lib32"] = lambda: torch.mm(A, Bt, out_dtype=torch.float32)
        except Exception:
            pass
        rounds = {k: [] for k in candidates}
        for _ in range(3):                       # the candidates take turns
            for k, fn in candidates.items():
                rounds[k].append(timed(fn))
        ours = statistics.median(rounds["ours"])
        lib = statistics.median(rounds["lib"])
        lib32 = statistics.median(rounds["lib32"]) if "lib32" in rounds else None
        flop = 2.0 * M * N * K
        out[f"{M}x{N}x{K}"] = {"us": round(ours, 2), "tflops": round(flop / ours / 1e6, 1),
                               "frac_of_mfma_peak": round(flop / (ours * 1e-6) / MFMA_F16_PEAK, 4),
                               "form": "256x256 tiles" if (M % 256 == 0 and N % 256 == 0 and (M // 256) * (N // 256) >= 256)
                               else "128x128 tiles",
                               "torch_matmul_us": round(lib, 2), "torch_matmul_tflops": round(flop / lib / 1e6, 1),
                               "torch_mm_fp32_out_us": None if lib32 is None else round(lib32, 2)}
    return out


def lc_leg(ta, torch, np, queries, be_name="stencil", be_label="stencil 512x512x64", be2_name="lbm"):
    """benchmark configuration 5: VGG16 batch 1 (224x224) as the latency-critical task, one best-effort kernel
    streamed block-slice by block-slice into its layers by TaskManager (block counts per layer measured by
    the manager's calibration pass, fused launch at most 10 % longer than the layer alone); query latency
    alone and co-located, and the best-effort work a query carries."""
    task = ta.LcTask("vgg16")
    tm = ta.TaskManager(task, be_name, be2_name)   # the second kernel only names the stage-2 pair (same family)
    tm.configure(qos_budget_ms=50.0, guard_ms=4.0, warmup=5, profile=min(500, queries), queries=queries, verbose=0)
    tm.set_calibration(True, 0.10)
    tm.set_calibration_variants(("default", "wave_256"))   # per layer: the pair's default form or the 512-thread one
    tm.set_end_to_end(min(500, queries))
    rep = tm.run("aker", second_stage=True)
    torch.cuda.synchronize()
    co = np.array(tm.latencies())
    solo = np.array(tm.latencies(solo=True))
    e2e = {k: np.array(tm.latencies(kind=k)) for k in ("e2e_solo", "e2e_colocated", "e2e_solo_wall", "e2e_colocated_wall",
                                                             "e2e_graph", "e2e_graph_wall")}
    be_total = ta.create_kernel(be_name).info()["ptb_end"]
    out = {"workload": f"configs[4]: VGG16 batch 1 224x224 (convs and FCs on tzgemm) + {be_label} "
                       "blocks co-located by TaskManager (Aker mode, calibrated block counts)",
           "queries": int(len(co)), "solo_queries": int(len(solo)),
           "solo_p50_ms": round(float(np.percentile(solo, 50)), 4),
           "solo_p99_ms": round(float(np.percentile(solo, 99)), 4),
           "colocated_p50_ms": round(float(np.percentile(co, 50)), 4),
           "colocated_p99_ms": round(float(np.percentile(co, 99)), 4),
           "qos_bound_ms": round(1.2 * float(np.percentile(solo, 99)), 4),
           "qos_budget_ms": 50.0,
           "mixed_launches_per_query": rep["mix_times"], "mixable_launches_per_query": rep["mixable_times"],
           "be_blocks_per_query": rep["be_blocks_executed"], "time_earned_ms_per_query": round(rep["time_earned_ms"], 4),
           "be_work_ms_per_query": round(rep["be_blocks_executed"] * rep["be1_solo_ms"] / be_total, 4),
           "be_kernel_passes_completed": rep["be_task_finish_num"],
           "lc_kernels_barred_from_fusion_at_end": tm.fusion_disabled(),
           "layers_calibrated_to_the_512_thread_form": sum(1 for v, n in zip(tm.calibrated_variants(), tm.calibrated_blocks())
                                                           if n > 0 and v == "wave_256")}
    out["p99_within_bound"] = bool(out["colocated_p99_ms"] <= out["qos_bound_ms"])
    # whole queries, one event pair (and the host clock) around all launches of a query, no
    # synchronisation between kernels; the figures above are sums of per-kernel intervals.  graph_*: the
    # solo query's launches recorded once and launched as one graph per query
    out["end_to_end"] = {"queries": int(len(e2e["e2e_solo"]))}
    for k, v in e2e.items():
        if len(v):
            out["end_to_end"][k[4:] + "_p50_ms"] = round(float(np.percentile(v, 50)), 4)
            out["end_to_end"][k[4:] + "_p99_ms"] = round(float(np.percentile(v, 99)), 4)
    if len(e2e["e2e_solo"]) and len(e2e["e2e_colocated"]):
        # what a client sees: the best-effort work a query carried (priced at the kernel's own rate) minus what
        # the query grew by, median to median -- no per-kernel synchronisation in either figure
        out["end_to_end"]["earned_ms_per_query"] = round(out["be_work_ms_per_query"] - float(
            np.percentile(e2e["e2e_colocated"], 50) - np.percentile(e2e["e2e_solo"], 50)), 4)
        bound = 1.2 * float(np.percentile(e2e["e2e_solo"], 99))
        out["end_to_end"]["qos_bound_ms"] = round(bound, 4)
        out["end_to_end"]["p99_within_bound"] = bool(np.percentile(e2e["e2e_colocated"], 99) <= bound)
    tm.close()
    task.close()
    return out


class PowerSampler:
    """socket power from the driver's hwmon file (microwatts), sampled from a thread while a leg runs; None
    where the file is absent or unreadable"""

    def __init__(self):
        import glob
        self.files = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")
        self.cap = None
        for f in glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap"):
            try:
                self.cap = int(open(f).read()) / 1e6
            except (OSError, ValueError):
                pass
        self.samples = []
        self.stop = False
        self.thread = None

    def usable(self):
        try:
            return bool(self.files) and int(open(self.files[0]).read()) > 0
        except (OSError, ValueError):
            return False

    def start(self):
        import threading

        def poll():
            while not self.stop:
                try:
                    self.samples.append((time.perf_counter(), int(open(self.files[0]).read()) / 1e6))
                except (OSError, ValueError):
                    pass
                time.sleep(0.02)
        self.thread = threading.Thread(target=poll, daemon=True)
        self.thread.start()

    def mean_between(self, t0, t1):
        w = [p for t, p in self.samples if t0 <= t <= t1]
        return sum(w) / len(w) if w else None

    def close(self):
        self.stop = True
        if self.thread:
            self.thread.join()


def power_leg(torch, job, seconds=1.5):
    """config 2's four jobs again, each looped for `seconds` with the socket power sampled every 20 ms (the first
    half second of a loop is left out: the sensor averages): is the fused launch held by the power limit?"""
    sampler = PowerSampler()
    if not sampler.usable():
        return None
    sampler.start()
    out = {"cap_w": sampler.cap, "sensor": "hwmon power1_input, 20 ms samples, loops of %.1f s" % seconds}
    for kind in ("gemm", "stencil", "serial", "fused"):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        n = 0
        while time.perf_counter() - t0 < seconds:
            job(kind)
            torch.cuda.synchronize()
            n += ITERATIONS
        t1 = time.perf_counter()
        w = sampler.mean_between(t0 + 0.5, t1)
        us = (t1 - t0) / n * 1e6
        out[kind] = {"mean_w": round(w, 0) if w else None, "us_per_iteration_incl_host": round(us, 2),
                     "mj_per_iteration": round(w * us * 1e-3, 2) if w else None}
    sampler.close()
    if out["fused"]["mean_w"] and sampler.cap:
        out["fused_frac_of_cap"] = round(out["fused"]["mean_w"] / sampler.cap, 3)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--variant", default=None, help="fused kernel variant (default: kinfo)")
    ap.add_argument("--grid", type=int, default=0, help="fused launch grid (default: kinfo gridsize x CUs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the other pairs (configs 3, 4) and the co-location latency leg (config 5)")
    ap.add_argument("--queries", type=int, default=1000, help="latency-critical queries of the co-location leg")
    ap.add_argument("--no-lc", action="store_true", help="skip the co-location latency legs (config 5)")
    ap.add_argument("--pairs", default="lbm,mriq,cp,mrif,sgemm,fft,cutcp,nn,hot3d,path,lava",
                    help="best-effort kernels of the other-pairs legs (comma separated); with a list of its own the "
                         "tzgemm shapes leg is skipped too (profiling runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU (no sharding, no collectives); use --gpus 1",
              file=sys.stderr)
        return 2

    import numpy as np
    import torch
    import tacker_amd as ta

    ta.init(0)
    M, N, K = GEMM_MNK
    nz, ny, nx = STENCIL_DIMS
    rng = np.random.default_rng(1337)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    B = rng.uniform(-1, 1, (N, K)).astype(np.float16)
    A0 = rng.uniform(0, 1, (nz, ny, nx)).astype(np.float32)
    c0, c1 = float(np.float32(1.0 / 6.0)), float(np.float32(1.0 / 6.0 / 6.0))

    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    dC = torch.zeros((M, N), device="cuda:0")
    g0 = torch.from_numpy(A0).cuda()
    g1 = g0.clone()
    stream = torch.cuda.current_stream()

    tiles = ta.tzgemm_grid_dim(M, N, K)[3]
    blocks = ta.stencil_blocks(nx, ny, nz)
    st_ori = ta.ori_stencil_create(c0, c1, g0, g1)
    st = ta.gptb_create(st_ori, 0, 0, 0, blocks)
    tz_ori = ta.ori_tzgemm_create(dA, dB, dC)
    tz = ta.gptb_create(tz_ori, 0, 0, 0, tiles)
    mix = ta.mix_create(st, tz, 0, blocks, 0, tiles, variant=args.variant, launch_grid=args.grid)

    def job(kind):
        for _ in range(ITERATIONS):
            if kind == "serial":
                tz.execute(stream)
                st.execute(stream)
            elif kind == "fused":
                mix.execute(stream)
            elif kind == "gemm":
                tz.execute(stream)
            elif kind == "stencil":
                st.execute(stream)
            if kind != "gemm":
                st_ori.swap_buffers()

    e0, e1 = ta.Event(), ta.Event()

    def timed(kind):
        torch.cuda.synchronize()
        e0.record(stream)
        job(kind)
        e1.record(stream)
        e1.synchronize()
        return e0.elapsed_ms(e1)

    for kind in ("gemm", "stencil", "serial", "fused"):
        for _ in range(args.warmup):
            job(kind)
    torch.cuda.synchronize()

    samples = {k: [] for k in ("gemm", "stencil", "serial", "fused")}
    torch.cuda.synchronize()
    t_wall = time.perf_counter()
    for _ in range(args.steps):                      # EXACTLY K timed steps of each form
        for kind in samples:
            samples[kind].append(timed(kind))
    torch.cuda.synchronize()
    t_wall = time.perf_counter() - t_wall
    ms = {k: trimmed_mean(v) for k, v in samples.items()}

    gemm_flop = 2.0 * M * N * K
    stencil_bytes = 2.0 * nx * ny * nz * 4                    # every cell read once, written once
    gemm_bytes = 2.0 * (M * K + N * K) + 4.0 * M * N          # A, B read once, C written once
    fused_bytes = stencil_bytes + gemm_bytes                  # algorithmic bytes of one fused launch
    fused_launch_s = ms["fused"] / ITERATIONS * 1e-3
    speedup = ms["serial"] / ms["fused"]
    info = mix.info()
    import statistics
    per_step = [a / b for a, b in zip(samples["serial"], samples["fused"])]   # serial and fused jobs alternate inside a step
    # Details first, headline last: a reader who keeps only the end of the line still has the metric,
    # the roofline and the summaries of every pair.
    out = {}
    if not args.no_extras:
        power = power_leg(torch, job)
        if power:
            out["power"] = power
        if args.pairs == ap.get_default("pairs"):
            out["tzgemm_shapes"] = gemm_leg(ta, torch, np, stream)
        out["other_pairs"] = {name: pair_leg(ta, torch, np, name, stream) for name in args.pairs.split(",") if name}
        if not args.no_lc:
            out["lc_colocation"] = lc_leg(ta, torch, np, args.queries)
            out["lc_colocation_mriq"] = lc_leg(ta, torch, np, args.queries, "mriq", "mri-q numK 2048, numX 262144")
            out["lc_colocation_fft"] = lc_leg(ta, torch, np, args.queries, "fft", "fft 10240 x 256 points")
            out["lc_colocation_nn"] = lc_leg(ta, torch, np, args.queries, "nn", "nn 655360000 records", "path")
    out["alone"] = {
        "tzgemm": {"avg_launch_us": round(ms["gemm"] * 10, 2),
                   "tflops": round(gemm_flop / (ms["gemm"] / ITERATIONS * 1e-3) / 1e12, 1),
                   "frac_of_mfma_peak": round(gemm_flop / (ms["gemm"] / ITERATIONS * 1e-3) / MFMA_F16_PEAK, 4)},
        "stencil": {"avg_launch_us": round(ms["stencil"] * 10, 2),
                    "gbps": round(stencil_bytes / (ms["stencil"] / ITERATIONS * 1e-3) / 1e9, 1),
                    "frac_of_hbm_peak": round(stencil_bytes / (ms["stencil"] / ITERATIONS * 1e-3) / HBM_PEAK, 4)}}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(A, B, A0, c0, c1)
    if "tzgemm_shapes" in out:
        # shape -> [tzgemm us, fraction of the MFMA peak, torch.matmul us (fp16 C), torch.mm us with an fp32 C]
        out["tzgemm_shapes_summary"] = {k: [v["us"], v["frac_of_mfma_peak"], v["torch_matmul_us"], v["torch_mm_fp32_out_us"]]
                                        for k, v in out["tzgemm_shapes"].items()}
    if "other_pairs" in out:
        # pair -> [whole kernel fused, slice at the kernel's rate, cursor (the scheduler's slices), GEMM us, best-effort us,
        #          serial us, fused us, slowest form the scheduler would pick]; speedups are serial / fused
        out["pairs_summary"] = {k: [v["speedup"], v.get("slice_speedup_at_kernel_rate"), v.get("cursor_speedup"),
                                    v["gemm_us"], v["be_us"], v["serial_us"], v["fused_us"],
                                    v["scheduler"]["slowest_form_it_would_pick"]]
                                for k, v in out["other_pairs"].items()}
        out["pairs_summary"]["stencil"] = [round(speedup, 4), None, None, round(ms["gemm"] * 10, 2),
                                           round(ms["stencil"] * 10, 2), round(ms["serial"] * 10, 2),
                                           round(ms["fused"] * 10, 2), round(speedup, 4)]
        losing = [k for k, v in out["pairs_summary"].items() if v[7] is not None and v[7] < 1.0]
        out["pairs_the_scheduler_would_fuse_at_a_loss"] = losing
    for key in ("lc_colocation", "lc_colocation_mriq", "lc_colocation_fft", "lc_colocation_nn"):
        if key in out:
            e = out[key]["end_to_end"]
            # [solo p50, solo p99, co-located p50, co-located p99, bound, within bound, ms earned per query,
            #  best-effort ms carried per query, fused layers, ms earned per query end to end]
            out[key + "_summary"] = [e.get("solo_p50_ms"), e.get("solo_p99_ms"), e.get("colocated_p50_ms"),
                                     e.get("colocated_p99_ms"), e.get("qos_bound_ms"), e.get("p99_within_bound"),
                                     out[key]["time_earned_ms_per_query"], out[key]["be_work_ms_per_query"],
                                     out[key]["mixed_launches_per_query"], e.get("earned_ms_per_query")]
    if "power" in out:
        # [GEMM alone W, stencil alone W, serial job W, fused job W, cap W]: is the fused launch held by the power limit?
        out["power_summary"] = [out["power"][k]["mean_w"] for k in ("gemm", "stencil", "serial", "fused")] + [out["power"]["cap_w"]]
    out.update({
        "wall_s_timed_region": round(t_wall, 3),
        "overlap_efficiency": round(max(ms["gemm"], ms["stencil"]) / ms["fused"], 4),
        "gemm_alone_ms_per_100": round(ms["gemm"], 4), "stencil_alone_ms_per_100": round(ms["stencil"], 4),
        "roofline_mfma": {"bound": "mfma", "achieved": round(gemm_flop / fused_launch_s / 1e12, 1),
                          "peak": MFMA_F16_PEAK / 1e12, "unit": "TFLOP/s",
                          "frac": round(gemm_flop / fused_launch_s / MFMA_F16_PEAK, 4),
                          "flop_per_launch": gemm_flop},
        "roofline": {"bound": "hbm", "achieved": round(fused_bytes / fused_launch_s / 1e9, 1),
                     "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(fused_bytes / fused_launch_s / HBM_PEAK, 4),
                     "traffic": FUSED_HBM_TRAFFIC_BYTES,
                     "kernel": "stencil_tzgemm_mix (one fused launch: 1 GEMM + 1 sweep)",
                     "algorithmic_bytes_per_launch": fused_bytes,
                     "avg_launch_us": round(fused_launch_s * 1e6, 2)},
        "config": {"workload": "configs[1]: fused tzgemm fp16 2048x2048x2048 + 7-point stencil fp32 "
                               "512x512x64, c0=1/6, c1=1/36, 100 iterations",
                   "fused_kernel": "tzgemm_stencil" + ("@" + args.variant if args.variant else " (kinfo default)"),
                   "fused_grid": info["grid"], "fused_block": info["block"], "device": ta.device_name()},
        "data": "synthetic (numpy default_rng(1337): A,B uniform[-1,1] -> f16; grid uniform[0,1])",
        "dtype": "f16 in / f32 accumulate (tzgemm), f32 (stencil)",
        "metric": "fused-pair speedup vs serial (tzgemm 2048^3 + stencil 512x512x64, 100 iterations)",
        "unit": "x", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        # value = trimmed mean of the serial job / trimmed mean of the fused job; per step: the ratio of the
        # two jobs of that step (they run back to back)
        "value_per_step": {"min": round(min(per_step), 4), "median": round(statistics.median(per_step), 4),
                           "max": round(max(per_step), 4)},
        "serial_ms_per_step": round(ms["serial"], 4), "ms_per_step": round(ms["fused"], 4),
        "value": round(speedup, 4),
    })
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
