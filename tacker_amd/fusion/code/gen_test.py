#!/usr/bin/env python3
"""Self-checking timing harness for the generated fused kernels (runs on the GPU).

Counterpart of ``fusion/code/gen_test.py`` of the reference together with the loop in
``gen_run.py`` :164-205 that compiles and runs one test program per fused candidate: each
program times the two GPTB kernels alone, times the fused kernel, compares the fused
outputs with the unfused ones (abs 1e-3 there) and prints ``[GPTB] ... took`` /
``[MIX] ... took`` lines the scripts scrape.  Here every candidate is already compiled into
the library and takes its ranges as launch parameters, so one process walks all of them:

  for each pair (tzgemm, be) and each variant the generator emitted
    check   fused outputs == outputs of the two GPTB kernels, bit for bit, on seeded inputs
            (a GEMM of 384x256x320 and a small instance of the vector kernel, full ranges and
            a partial range)
    time    GEMM alone, vector kernel alone, both serially, fused -- at the benchmark sizes,
            trimmed mean of --rounds timing loops of --launches launches

    python gen_test.py                      # table for every pair and variant
    python gen_test.py --pairs stencil      # one pair
    python gen_test.py --write-default      # also store the fastest correct variant per pair
                                            # in defaults.json (then gen_run.py + make)
Exit status 1 if any candidate's outputs differ.
"""
import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.abspath(os.path.join(HERE, "..", "..", ".."))
sys.path.insert(0, HERE)
sys.path.insert(0, ROOT)

import gen_run  # noqa: E402

DEFAULTS = os.path.join(HERE, "defaults.json")


def make_inputs(np, torch, ta, be, small):
    """Device buffers of one vector kernel: (ori kernel object, blocks, [output tensors])."""
    rng = np.random.default_rng(1337)
    if be == "stencil":
        shape = (6, 20, 200) if small else (64, 512, 512)
        a0 = torch.from_numpy(rng.uniform(0, 1, shape).astype(np.float32)).cuda()
        out = a0.clone()
        c0 = float(np.float32(1.0 / 6.0))
        c1 = float(np.float32(1.0 / 36.0))
        return ta.ori_stencil_create(c0, c1, a0, out), ta.stencil_blocks(shape[2], shape[1], shape[0]), [out]
    if be == "lbm":
        sx, sy, sz = (120, 6, 5) if small else (120, 120, 150)
        cells = sx * sy * sz
        w = np.array([1 / 3] + [1 / 18] * 6 + [1 / 36] * 12, np.float32)
        g = np.zeros((20, cells), np.float32)
        g[:19] = w[:, None] + rng.uniform(0, 1e-3, (19, cells)).astype(np.float32)
        g[19] = (rng.uniform(0, 1, cells) < 0.05).astype(np.uint32).view(np.float32)
        src = torch.from_numpy(g.reshape(-1)).cuda()
        dst = torch.zeros_like(src)
        return ta.ori_lbm_create(src, dst, sx, sy, sz), sy * sz, [dst]
    if be == "mriq":
        numK, numX = (256, 2048) if small else (2048, 262144)
        k = rng.uniform(-0.5, 0.5, (numK, 3)).astype(np.float32)
        phi = rng.uniform(0, 1, (2, numK)).astype(np.float32)
        kv = np.concatenate([k, (phi[0] * phi[0] + phi[1] * phi[1])[:, None]], 1).astype(np.float32)
        ta.mriq_set_kvalues(kv)
        xyz = [torch.from_numpy(rng.uniform(-0.5, 0.5, numX).astype(np.float32)).cuda() for _ in range(3)]
        Qr, Qi = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
        return ta.ori_mriq_create(numK, xyz[0], xyz[1], xyz[2], Qr, Qi), ta.mriq_blocks(numK, numX), [Qr, Qi]
    if be == "mrif":
        numK, numX = (256, 2048) if small else (2048, 262144)
        k = rng.uniform(-0.5, 0.5, (numK, 3)).astype(np.float32)
        phi = rng.uniform(0, 1, (2, numK)).astype(np.float32)
        d = rng.uniform(0, 1, (2, numK)).astype(np.float32)
        rho = np.stack([phi[0] * d[0] + phi[1] * d[1], phi[0] * d[1] - phi[1] * d[0]], 1)
        ta.mrif_set_kvalues(np.concatenate([k, rho], 1).astype(np.float32))
        xyz = [torch.from_numpy(rng.uniform(-0.5, 0.5, numX).astype(np.float32)).cuda() for _ in range(3)]
        outR, outI = torch.zeros(numX, device="cuda:0"), torch.zeros(numX, device="cuda:0")
        return ta.ori_mrif_create(numK, xyz[0], xyz[1], xyz[2], outR, outI), ta.mrif_blocks(numK, numX), [outR, outI]
    if be == "cp":
        ta.cp_set_atoms(ta.cp_initatoms(4000)[1:65], 0.0)
        shape = (32, 512) if small else (4096, 4096)
        grid = torch.zeros(shape, device="cuda:0")
        return ta.ori_cp_create(64, 0.1, grid), ta.cp_blocks(shape[1], shape[0]), [grid]
    if be == "fft":
        batches = 40 if small else 10240
        data = torch.from_numpy(rng.uniform(-1, 1, (batches, 256, 2)).astype(np.float32)).cuda()
        return ta.ori_fft_create(data), batches, [data]
    if be == "cutcp":
        n, count = (24, 400) if small else (208, 70000)
        atoms = np.empty((count, 4), np.float32)
        atoms[:, :3] = rng.uniform(0, (n - 1) * 0.5, (count, 3))
        atoms[:, 3] = rng.uniform(0.1, 1, count) * rng.choice([-1, 1], count)
        # the benchmark instance computes the two lowest layers of regions of the 208^3 lattice
        inp = ta.CutcpInput(atoms, (0, 0, 0), n, n, n, 0.5, 12.0, regions=None if small else (26, 26, 2))
        return ta.ori_cutcp_create(inp, 144.0, 0.006944), inp.blocks(), [inp.energies]
    if be == "nn":
        records = 256 * 37 + 5 if small else 256 * 2560000
        loc = torch.rand((records, 2), device="cuda:0") * 90.0
        dist = torch.zeros(records, device="cuda:0")
        return ta.ori_nn_create(loc, dist, 30.0, 90.0), ta.nn_blocks(records), [dist]
    if be == "hot3d":
        nx, ny, nz = (128, 16, 4) if small else (16384, 8192, 8)
        power = torch.rand((nz, ny, nx), device="cuda:0") * 0.01
        t_in = torch.rand((nz, ny, nx), device="cuda:0") * 20.0 + 320.0
        t_out = torch.zeros((nz, ny, nx), device="cuda:0")
        return ta.ori_hot3d_create(power, t_in, t_out), ta.hot3d_blocks(nx, ny), [t_out]
    if be == "lava":
        boxes1d = 2 if small else 60
        n = 100 * boxes1d ** 3
        rv = torch.rand((n, 4), device="cuda:0") * 0.9 + 0.1
        qv = torch.rand(n, device="cuda:0") * 0.9 + 0.1
        fv = torch.zeros((n, 4), device="cuda:0")
        return ta.ori_lava_create(0.5, rv, qv, fv), ta.lava_blocks(boxes1d), [fv]
    if be == "path":
        cols, height = (700, 60) if small else (1200, 125)
        wall = torch.from_numpy(rng.integers(0, 10, (height, cols), dtype=np.int32)).cuda()
        src = torch.from_numpy(rng.integers(0, 10, cols, dtype=np.int32)).cuda()
        out = torch.zeros(cols, dtype=torch.int32, device="cuda:0")
        return ta.ori_path_create(height, wall, src, out), ta.path_blocks(cols, height), [out]
    if be == "sgemm":
        M, N, K = (256, 48, 300) if small else (4096, 4128, 4064)
        A = torch.from_numpy(rng.uniform(0, 1, (K, M)).astype(np.float32)).cuda()
        B = torch.from_numpy(rng.uniform(0, 1, (K, N)).astype(np.float32)).cuda()
        Cm = torch.zeros((N, M), device="cuda:0")
        return ta.ori_sgemm_create(A, B, Cm), ta.sgemm_blocks(M, N, K), [Cm]
    raise SystemExit(f"unknown kernel {be}")


def make_gemm(np, torch, ta, M, N, K):
    rng = np.random.default_rng(7)
    A = torch.from_numpy(rng.uniform(-1, 1, (M, K)).astype(np.float16)).cuda()
    B = torch.from_numpy(rng.uniform(-1, 1, (N, K)).astype(np.float16)).cuda()
    Cm = torch.zeros((M, N), device="cuda:0")
    tiles = (M // 64) * (N // 64)
    return ta.ori_tzgemm_create(A, B, Cm), tiles, Cm


def check_variant(np, torch, ta, be, variant):
    """fused == unfused, bit for bit, over full ranges and over a partial range"""
    ok = True
    for part in (False, True):
        be_ori, nblk, outs = make_inputs(np, torch, ta, be, small=True)
        tz_ori, tiles, Cm = make_gemm(np, torch, ta, 384, 256, 320)
        b0, b1 = (nblk // 3, nblk - 1) if part else (0, nblk)
        if part and be == "sgemm":
            b0 = 0   # its later k parts go on from a workspace the comparison does not restore: start with part 0
        t0, t1 = (2, tiles - 3) if part else (0, tiles)
        snap = [o.clone() for o in outs]
        be_k = ta.gptb_create(be_ori, 0, 0, b0, b1)
        tz_k = ta.gptb_create(tz_ori, 0, 0, t0, t1)
        Cm.fill_(-7.0)
        be_k.execute()
        tz_k.execute()
        torch.cuda.synchronize()
        want = [o.clone() for o in outs] + [Cm.clone()]
        for o, s in zip(outs, snap):
            o.copy_(s)
        Cm.fill_(-7.0)
        be_full = ta.gptb_create(be_ori, 0, 0, 0, nblk)
        tz_full = ta.gptb_create(tz_ori, 0, 0, 0, tiles)
        mix = ta.mix_create(be_full, tz_full, b0, b1, t0, t1, variant=variant)
        mix.execute()
        torch.cuda.synchronize()
        got = list(outs) + [Cm]
        same = all(torch.equal(g.view(torch.int32), w.view(torch.int32)) for g, w in zip(got, want))
        ok = ok and same and ta.spin_fail_flag() == 0
    return ok


def time_variants(np, torch, ta, be, variants, launches, rounds):
    be_ori, nblk, _ = make_inputs(np, torch, ta, be, small=False)
    M, N, K = (4096, 4096, 1024) if be == "lbm" else (2048, 2048, 2048)
    tz_ori, tiles, _ = make_gemm(np, torch, ta, M, N, K)
    be_k = ta.gptb_create(be_ori, 0, 0, 0, nblk)
    tz_k = ta.gptb_create(tz_ori, 0, 0, 0, tiles)
    e0, e1 = ta.Event(), ta.Event()

    def timed(fn):
        torch.cuda.synchronize()
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        e1.synchronize()
        return e0.elapsed_ms(e1) / launches * 1e3

    def serial():
        tz_k.execute()
        be_k.execute()

    cases = {"tzgemm": tz_k.execute, be: be_k.execute, "serial": serial}
    for v in variants:
        cases[v] = ta.mix_create(be_k, tz_k, 0, nblk, 0, tiles, variant=v).execute
    samples = {name: [] for name in cases}
    for _ in range(rounds + 1):                 # first round is warm-up
        for name, fn in cases.items():
            samples[name].append(timed(fn))
    out = {}
    for name, v in samples.items():
        v = sorted(v[1:])
        if len(v) >= 4:
            v = v[1:-1]
        out[name] = sum(v) / len(v)
    return out, (M, N, K)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--pairs", nargs="*", default=gen_run.BE_KERNELS)
    ap.add_argument("--launches", type=int, default=200)
    ap.add_argument("--rounds", type=int, default=4)
    ap.add_argument("--write-default", action="store_true")
    args = ap.parse_args()

    import numpy as np
    import torch
    import tacker_amd as ta

    ta.init(0)
    failed = False
    best = {}
    for be in args.pairs:
        variants = []
        for cand in gen_run.pair_candidates(be):
            variants.append(f"wg_{cand[1]}_{cand[2]}" if cand[0] == "wg" else f"wave_{cand[1]}")
        good = []
        for v in variants:
            ok = check_variant(np, torch, ta, be, v)
            print(f"[CHECK] tzgemm_{be}@{v}: fused outputs {'match' if ok else 'DIFFER from'} the unfused kernels",
                  flush=True)
            if ok:
                good.append(v)
            else:
                failed = True
        t, mnk = time_variants(np, torch, ta, be, good, args.launches, args.rounds)
        print(f"[GPTB] tzgemm {mnk[0]}x{mnk[1]}x{mnk[2]} took {t['tzgemm'] / 1e3:.6f} ms")
        print(f"[GPTB] {be} took {t[be] / 1e3:.6f} ms")
        print(f"[SERIAL] tzgemm + {be} took {t['serial'] / 1e3:.6f} ms")
        for v in good:
            print(f"[MIX] tzgemm_{be} {v} took {t[v] / 1e3:.6f} ms   speedup over serial {t['serial'] / t[v]:.3f}",
                  flush=True)
        if good:
            best[be] = min(good, key=lambda v: t[v])
            print(f"[BEST] tzgemm_{be}: {best[be]}\n", flush=True)
    if args.write_default and best:
        dflt = json.load(open(DEFAULTS))
        for be, v in best.items():
            dflt[f"tzgemm_{be}"]["variant"] = v
        with open(DEFAULTS, "w") as f:
            json.dump(dflt, f, indent=2)
            f.write("\n")
        print("updated", DEFAULTS, "- now run gen_run.py and rebuild")
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
