#!/usr/bin/env python3
"""Measure the load ratio of every fused pair on the GPU and write it into the kernel-info
defaults: for a tzgemm of reduction length K, how many best-effort blocks per GEMM tile
should ride along in one fused launch.

Stands for the reference's load-ratio experiments (fusion/expr_load_ratio/*.py: sweep the
best-effort block count of a fused kernel, keep the count at which both halves finish
together) and the table they feed (`block_ratio` and the per-K entries TaskManager looks up,
src/TaskManager.cu:593-600).  Instead of recompiling one .cu per point, the fused kernels of
this build take their ranges as launch parameters, so a sweep is a loop of launches.

Two steps, because the GPU box and the build tree are different places:
    python profile_ratio.py --measure out.json          # on the GPU
    python profile_ratio.py --apply out.json            # rewrites defaults.json; then gen_run.py
Method per (pair, K): GEMM 2048 x 2048 x K (1024 tiles, one 128x128 macro tile per CU).
t_gemm = the GEMM's own kernel alone, t_be = the best-effort kernel alone (all N blocks).
For nb on a ladder of block counts (every launch carrying the next nb positions of the kernel, so that
no launch finds its data left in the caches by the one before), earned(nb) = t_gemm + t_be * nb / N - t_fused(nb)
is the time one fused launch saves over the two serial launches (the quantity TaskManager
credits, src/TaskManager.cu:626-640); a count qualifies only if it earns at least min_gain
(3 %) of those serial launches, so that a pair within the noise of breaking even is not fused; the ladder runs N/1024, N/512, ..., N/64 (from N/65536 for grids of
a million positions and more), then N/32, 2N/32, ..., N and stops once a launch is twice as long as allowed.  The ratio is nb / 1024 for the nb with the largest
earned time among those whose launch stays within (1 + stretch) * t_gemm, i.e. the
latency-critical GEMM is never stretched by more than that factor; 0 if nothing earns.
Per pair also `whole_kernel_gain`: the 2048^3 GEMM and the whole best-effort kernel as two launches
over the one fused launch that carries both; below 1 the scheduler's Tacker mode, which would let
the whole kernel ride, carries the slice of the table instead.
"""
import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.abspath(os.path.join(HERE, "..", "..", ".."))
DEFAULTS = os.path.join(HERE, "defaults.json")
# reduction lengths of the VGG16 batch-1 layers after padding to 128, plus the benchmark's
K_LADDER = (128, 640, 1152, 2048, 2304, 4096, 4608)
PAIRS = ("stencil", "lbm", "mriq", "cp", "mrif", "sgemm", "fft", "cutcp", "nn", "hot3d", "path", "lava")
TILES = 1024
LADDER = 32          # best-effort block counts tried: N/1024, N/512, ..., N/64, then N/32, 2N/32, ..., N


def ladder(be_total, points=0):
    """points > 0: that many counts only, spread geometrically from N/64 to N (a quick check of the
    method); otherwise
    ascending block counts: a geometric run-up for kernels whose 1/32 is already longer than a GEMM
    (sgemm: 2 ms for 528384 positions; from 1/65536 for grids of a million positions and more -- lavaMD:
    43 ms for 5832000), then the linear ladder"""
    if points > 0:
        steps = max(points - 1, 1)
        return sorted({max(1, int(round(be_total / 64 ** ((steps - i) / steps)))) for i in range(points)})
    deepest = 17 if be_total >= 1 << 20 else 11
    counts = {be_total >> j for j in range(6, deepest)} | {be_total * step // LADDER for step in range(1, LADDER + 1)}
    return sorted(c for c in counts if c > 0)


def measure(out_path, stretch, launches, pairs=PAIRS, k_ladder=K_LADDER, ladder_points=0, min_gain=0.03):
    sys.path.insert(0, ROOT)
    import torch
    import tacker_amd as ta

    ta.init(0)
    e0, e1 = ta.Event(), ta.Event()

    def timed(kernel):
        # Warm up for at least 5 ms of the kernel's own work before timing: after an allocation or a
        # copy the GPU is back at idle clocks, and a kernel of 20 us timed over its first hundred
        # launches reads up to a quarter too long -- which, for the GEMM alone, would be booked as
        # time the fused launch "earns".
        torch.cuda.synchronize()
        e0.record()
        for _ in range(3):
            kernel.execute()
        e1.record()
        e1.synchronize()
        est_us = max(e0.elapsed_ms(e1) / 3 * 1e3, 1.0)
        for _ in range(int(min(max(10, 5000.0 / est_us), 4 * launches))):
            kernel.execute()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(launches):
            kernel.execute()
        e1.record()
        e1.synchronize()
        return e0.elapsed_ms(e1) / launches * 1e3

    class Cursor:
        """the fused kernel carrying nb block positions a launch, every launch the next nb of the kernel's
        range (as TaskManager's cursor does): launched over one range again and again, a kernel that streams
        its data would find it in the caches and its slice would look cheaper than it is"""

        def __init__(self, mix, nb, total):
            self.mix, self.nb, self.total, self.lo = mix, nb, total, 0

        def execute(self):
            if self.lo + self.nb > self.total:
                self.lo = 0
            self.mix.set_range(self.lo, self.lo + self.nb, 0, TILES)
            self.mix.execute()
            self.lo += self.nb

    result = {"stretch": stretch, "min_gain": min_gain, "tiles": TILES, "device": ta.device_name(), "pairs": {}}
    for be_name in pairs:
        be = ta.create_kernel(be_name)
        be_total = be.info()["ptb_end"]
        be_us = timed(be)
        table = {}
        for K in k_ladder:
            A = (torch.rand((2048, K), device="cuda") * 2 - 1).half()
            B = (torch.rand((2048, K), device="cuda") * 2 - 1).half()
            Cm = torch.zeros((2048, 2048), device="cuda")
            tz = ta.gptb_create(ta.ori_tzgemm_create(A, B, Cm), 0, 0, 0, TILES)
            mix = ta.mix_create(be, tz, 0, 0, 0, TILES)
            t_gemm = timed(tz)           # the serial side: the GEMM's own kernel ...
            t0 = timed(mix)              # ... which the fused kernel carrying nothing does not quite match
            t_gemm = min(t_gemm, timed(tz))
            best = {"blocks": 0, "earned_us": 0.0, "fused_us": t0}
            for nb in ladder(be_total, ladder_points):
                t = timed(Cursor(mix, nb, be_total))
                serial = t_gemm + be_us * nb / be_total
                earned = serial - t
                if t <= (1 + stretch) * t_gemm and earned >= min_gain * serial and earned > best["earned_us"]:
                    best = {"blocks": nb, "earned_us": earned, "fused_us": t}
                if t > 2 * (1 + stretch) * t_gemm:      # more blocks only make the launch longer
                    break
            table[str(K)] = {"blocks": best["blocks"], "ratio": round(best["blocks"] / TILES, 4),
                             "gemm_us": round(t_gemm, 2), "gemm_in_fused_us": round(t0, 2), "fused_us": round(best["fused_us"], 2),
                             "earned_us": round(best["earned_us"], 2)}
            print(f"tzgemm_{be_name} K={K}: GEMM {t_gemm:.1f} us ({t0:.1f} in the fused kernel), best {best['blocks']} of {be_total} blocks "
                  f"(fused {best['fused_us']:.1f} us, earns {best['earned_us']:.1f} us) "
                  f"-> ratio {best['blocks'] / TILES:.4f}", flush=True)
        # the whole best-effort kernel in one fused launch with the 2048^3 GEMM against the two launches
        # (what TaskManager's Tacker mode does); the two are timed back to back, as they would run
        A = (torch.rand((2048, 2048), device="cuda") * 2 - 1).half()
        B = (torch.rand((2048, 2048), device="cuda") * 2 - 1).half()
        Cm = torch.zeros((2048, 2048), device="cuda")
        tz = ta.gptb_create(ta.ori_tzgemm_create(A, B, Cm), 0, 0, 0, TILES)
        whole = ta.mix_create(be, tz, 0, be_total, 0, TILES)

        class Serial:
            def execute(self):
                tz.execute()
                be.execute()

        serial_us, whole_us = timed(Serial()), timed(whole)
        print(f"tzgemm_{be_name} whole kernel: serial {serial_us:.1f} us, fused {whole_us:.1f} us "
              f"-> gain {serial_us / whole_us:.4f}", flush=True)
        result["pairs"]["tzgemm_" + be_name] = {"be_total_blocks": be_total, "be_solo_us": round(be_us, 2),
                                                "by_k": table,
                                                "whole_kernel": {"serial_us": round(serial_us, 2),
                                                                 "fused_us": round(whole_us, 2),
                                                                 "gain": round(serial_us / whole_us, 4)}}
    with open(out_path, "w") as f:
        json.dump(result, f, indent=1)
    print("wrote", out_path)


def apply(in_path):
    with open(in_path) as f:
        meas = json.load(f)
    with open(DEFAULTS) as f:
        dflt = json.load(f)
    for key, m in meas["pairs"].items():
        if key not in dflt:
            raise SystemExit(f"{DEFAULTS} has no entry {key}: add the pair to the generator first")
        entry = dflt[key]
        ratios = {k: v["ratio"] for k, v in m["by_k"].items()}
        # A pair's earnings change smoothly with K.  A K whose count clears the min_gain bar while both of
        # its neighbours on the ladder earn nothing cleared it by the noise of the timings: not fused.
        ks = sorted(ratios, key=int)
        for i, k in enumerate(ks):
            around = [ratios[ks[j]] for j in (i - 1, i + 1) if 0 <= j < len(ks)]
            if ratios[k] > 0 and around and not any(r > 0 for r in around):
                print(f"{key}: K = {k} earns alone among its neighbours ({m['by_k'][k]['ratio']}): taken as noise, ratio 0")
                ratios[k] = 0.0
        entry["ratio_by_k"] = ratios
        entry["block_ratio"] = ratios["4096"]
        if "whole_kernel" in m:
            entry["whole_kernel_gain"] = m["whole_kernel"]["gain"]
    dflt["ratio_provenance"] = {"stretch": meas["stretch"], "min_gain": meas.get("min_gain", 0.0), "device": meas["device"],
                                "method": "profile_ratio.py: GEMM 2048x2048xK; best-effort block count with "
                                          "the largest time earned over serial launches (at least min_gain of "
                                          "them) whose fused launch stays within (1+stretch) of the GEMM "
                                          "alone, divided by 1024 tiles; a K that earns while both "
                                          "neighbouring K of the ladder do not is set to 0"}
    with open(DEFAULTS, "w") as f:
        json.dump(dflt, f, indent=2)
        f.write("\n")
    print("updated", DEFAULTS, "- now run gen_run.py and rebuild")


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--measure", metavar="OUT.json")
    ap.add_argument("--apply", metavar="IN.json")
    ap.add_argument("--stretch", type=float, default=1.0,
                    help="largest tolerated stretch of the GEMM's launch (1.0 = at most twice as long)")
    ap.add_argument("--min-gain", type=float, default=0.03,
                    help="a block count qualifies only if the fused launch saves this fraction of the serial launches")
    ap.add_argument("--launches", type=int, default=100)
    ap.add_argument("--k-ladder", default=",".join(str(k) for k in K_LADDER), help="reduction lengths to measure at")
    ap.add_argument("--ladder-points", type=int, default=0,
                    help="measure only this many block counts per K (N/64 .. N); 0 = the full ladder")
    ap.add_argument("--pairs", default=",".join(PAIRS),
                    help="best-effort kernels to measure (comma separated); --apply only touches those measured")
    args = ap.parse_args()
    if args.measure:
        measure(args.measure, args.stretch, args.launches, tuple(args.pairs.split(",")),
                tuple(int(k) for k in args.k_ladder.split(",")), args.ladder_points, args.min_gain)
    elif args.apply:
        apply(args.apply)
    else:
        ap.error("one of --measure / --apply")


if __name__ == "__main__":
    main()
