#!/usr/bin/env python3
"""Extracts the fusion-candidate lists the reference ships as data
(fusion/code/log.txt, fusion/code/mix_kernel_info.txt) and the names of its
generated fused kernels (fusion/mix_kernel/*.cu) into generator_candidates.json.

Run in the authoring container, where the reference tree is mounted:
    python tests/golden/make_generator_fixtures.py /root/reference
The JSON holds numbers and file names only (no source text).
"""
import json
import os
import re
import sys


def main(ref):
    out = {"log": {}, "mix_kernel_info": {}, "mix_kernel_files": []}
    cur = None
    for line in open(os.path.join(ref, "fusion/code/log.txt")):
        m = re.match(r"candidates for (\w+?)_(\w+):", line)
        if m:
            cur = f"{m.group(1)} {m.group(2)}"
            out["log"][cur] = []
            continue
        m = re.match(r"kernel1_num:\s+(\d+) kernel2_num:\s+(\d+) blks_per_sm:\s+(\d+) reg used:\s+(\d+) "
                     r"sm used:\s+(\d+) thread used:\s+(\d+)", line)
        if m:
            out["log"][cur].append([int(x) for x in m.groups()])
    pair = main_k = None
    for line in open(os.path.join(ref, "fusion/code/mix_kernel_info.txt")):
        m = re.match(r"kernel pair:\s+(\w+) (\w+)", line)
        if m:
            pair = (m.group(1), m.group(2))
            continue
        m = re.match(r"- (\w+) as main kernel:", line)
        if m:
            main_k = m.group(1)
            out["mix_kernel_info"][f"{pair[0]} {pair[1]} {main_k}"] = []
            continue
        m = re.match(r"-- \w+_num: (\d+) \w+_num: (\d+) blks_per_sm: (\d+) reg used: (\d+) smem used: (\d+) "
                     r"thread used: (\d+)", line)
        if m:
            out["mix_kernel_info"][f"{pair[0]} {pair[1]} {main_k}"].append([int(x) for x in m.groups()])
    out["mix_kernel_files"] = sorted(f[:-3] for f in os.listdir(os.path.join(ref, "fusion/mix_kernel"))
                                     if f.endswith(".cu"))
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "generator_candidates.json")
    json.dump(out, open(dst, "w"), indent=0, separators=(",", ":"))
    print(f"wrote {dst}: {len(out['log'])} log pairs, {len(out['mix_kernel_info'])} info entries, "
          f"{len(out['mix_kernel_files'])} file names")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
