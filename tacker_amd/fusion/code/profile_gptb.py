#!/usr/bin/env python3
"""Time every best-effort kernel's GPTB launch over a ladder of block counts and of launch sizes.

Stands for the reference's block-count profile (fusion/code/gptb_profile.py with the programs of
fusion/gptb_profile/: one generated .cu per kernel and block count, compiled and run, its time
logged).  The GPTB kernels of this build take their range and their launch grid as launch
parameters, so the sweep is a loop of launches over the benchmark-size instances gen_test.py builds:

    python profile_gptb.py --measure out.json [--kernels stencil,lbm,...]

Per kernel it records
  * time of the whole range for 1, 2, 4, 8, 16 and 32 persistent workgroups per CU (what
    data.py's solo_ptb_blks should name), and
  * time of the ranges [0, n) for n on a ladder up to the whole grid at the kernel's kinfo launch
    size, beside what TaskManager's predictor says for them (whole time * n / N,
    src/TaskManager.cu:593-600), with the largest deviation of the two.
"""
import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.abspath(os.path.join(HERE, "..", "..", ".."))
sys.path.insert(0, HERE)
import gen_run  # noqa: E402
import gen_test  # noqa: E402

PER_CU = (1, 2, 4, 8, 16, 32)
LADDER = (1 / 64, 1 / 32, 1 / 16, 1 / 8, 1 / 4, 1 / 2, 3 / 4, 1.0)


def measure(out_path, kernels, launches):
    sys.path.insert(0, ROOT)
    import torch
    import tacker_amd as ta

    import numpy as np
    ta.init(0)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    e0, e1 = ta.Event(), ta.Event()
    outs, start_values = [], []

    def timed(kernel, n):
        for o, v in zip(outs, start_values):      # kernels that accumulate start every point from the same values
            o.copy_(v)
        kernel.execute()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(n):
            kernel.execute()
        e1.record()
        e1.synchronize()
        return e0.elapsed_ms(e1) / n * 1e3

    result = {"device": ta.device_name(), "kernels": {}}
    for name in kernels:
        ori, total, outs = gen_test.make_inputs(np, torch, ta, name, small=False)
        start_values = [o.clone() for o in outs]
        k = ta.gptb_create(ori, 0, 0, 0, total)           # launch size from kinfo
        info = k.info()
        block = info["block"]
        whole = timed(k, min(launches, 5))
        n = max(2, min(launches, int(2e5 / max(whole, 1.0))))      # about 0.2 s a point
        by_size = {}
        for per_cu in PER_CU:
            g = ta.gptb_create(ori, cus * per_cu, block, 0, total)
            by_size[str(per_cu)] = round(timed(g, n), 2)
        whole = timed(k, n)
        by_count, worst = {}, 0.0
        for frac in LADDER:
            nb = max(1, int(total * frac))
            k.set_range(0, nb)
            t = timed(k, n)
            predicted = whole * nb / total
            by_count[str(nb)] = {"us": round(t, 2), "predicted_us": round(predicted, 2)}
            if frac >= 1 / 8:
                worst = max(worst, abs(t - predicted) / predicted)
        k.set_range(0, total)
        result["kernels"][name] = {"blocks": total, "blocksize": block, "kinfo_workgroups_per_cu": info["grid"] // cus,
                                   "whole_us": round(whole, 2), "whole_us_by_workgroups_per_cu": by_size,
                                   "by_block_count": by_count,
                                   "largest_deviation_from_linear_from_an_eighth_up": round(worst, 4)}
        best = min(by_size, key=by_size.get)
        print(f"{name}: {total} blocks, {whole:.1f} us at {info['grid'] // cus} workgroups a CU; by workgroups a CU "
              f"{by_size} (best {best}); linear model off by at most {worst * 100:.1f} % from 1/8 of the grid up",
              flush=True)
    with open(out_path, "w") as f:
        json.dump(result, f, indent=1)
    print("wrote", out_path)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--measure", metavar="OUT.json", required=True)
    ap.add_argument("--kernels", default=",".join(gen_run.BE_KERNELS))
    ap.add_argument("--launches", type=int, default=20)
    args = ap.parse_args()
    measure(args.measure, [k for k in args.kernels.split(",") if k], args.launches)


if __name__ == "__main__":
    main()
