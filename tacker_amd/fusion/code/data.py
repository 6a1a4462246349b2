"""Kernel resource tables and the fusion-candidate rule.

Restates ``fusion/code/data.py`` of the reference (resource table :22-35,
``fuse_kernel_info`` :48-69) with the budgets as an argument, so the same rule
serves the reference's Turing SM numbers (used by the tests to reproduce the
candidate lists the reference ships in ``fusion/code/mix_kernel_info.txt``) and
the CDNA4 compute-unit numbers used for the gfx950 build.
"""
from collections import namedtuple
from math import gcd

Budget = namedtuple("Budget", "registers thread_slots shared_memory")

# One Turing SM as the reference assumes it (fusion/code/data.py:22-24).
TURING_SM = Budget(registers=65536, thread_slots=1024, shared_memory=65536)
# One CDNA4 compute unit: 4 SIMDs x 512 VGPRs x 64 lanes, 8 wave64 per SIMD,
# 160 KiB LDS.
CDNA4_CU = Budget(registers=4 * 512 * 64, thread_slots=4 * 8 * 64, shared_memory=160 * 1024)

WAVE_SIZE = 64
CU_NUM = 256
XCD_NUM = 8

# The reference's table (nvcc -Xptxas -v on sm_75), fusion/code/data.py:25-35.
# cp carries solo_ptb_blks = 6 here: the value the shipped candidate lists were
# generated with (the comment at :26 says "6 for mix").
REFERENCE_KERNEL_INFO = {
    "cp": {"register": 39, "shared_memory": 0, "blocksize": 128, "solo_ptb_blks": 6},
    "cutcp": {"register": 42, "shared_memory": 4096, "blocksize": 128, "solo_ptb_blks": 6},
    "fft": {"register": 33, "shared_memory": 2048, "blocksize": 128, "solo_ptb_blks": 3},
    "lbm": {"register": 61, "shared_memory": 0, "blocksize": 128, "solo_ptb_blks": 1},
    "mrif": {"register": 32, "shared_memory": 0, "blocksize": 256, "solo_ptb_blks": 3},
    "mriq": {"register": 31, "shared_memory": 0, "blocksize": 256, "solo_ptb_blks": 4},
    "sgemm": {"register": 64, "shared_memory": 512, "blocksize": 128, "solo_ptb_blks": 4},
    "tpacf": {"register": 41, "shared_memory": 13312, "blocksize": 256, "solo_ptb_blks": 3},
    "stencil": {"register": 38, "shared_memory": 1024, "blocksize": 128, "solo_ptb_blks": 3},
}

# gfx950 roles.  register = VGPRs per lane of the role compiled alone (from the
# code-object metadata, see gen_run.py --resources), shared_memory = LDS bytes
# per role instance, blocksize = threads of one role instance (a multiple of the
# 64-wide wavefront), solo_ptb_blks = role instances per CU of the plain GPTB
# launch, ori_blks = blocks of the reference-shaped natural grid at the
# benchmark's problem size.
KERNEL_INFO = {
    "tzgemm": {"register": 160, "shared_memory": 131072, "blocksize": 256, "solo_ptb_blks": 1},
    # 1024 blocks of 64 x 4 columns x 8 runs of 8 centre planes
    "stencil": {"register": 48, "shared_memory": 0, "blocksize": 256, "solo_ptb_blks": 8,
                "ori_blks": 8192},
    # 67.4 us with 16 workgroups a CU, 69.9 with 8 (profile_gptb.py)
    "lbm": {"register": 64, "shared_memory": 0, "blocksize": 256, "solo_ptb_blks": 16,
            "ori_blks": 18000},
    # 1024 blocks of 256 voxels x 16 chunks of 128 k records
    "mriq": {"register": 40, "shared_memory": 0, "blocksize": 256, "solo_ptb_blks": 8,
             "ori_blks": 16384},
    # 1024 blocks of 256 voxels x 16 chunks of 128 k records
    "mrif": {"register": 44, "shared_memory": 0, "blocksize": 256, "solo_ptb_blks": 8,
             "ori_blks": 16384},
    # 32 x 258 blocks of 128 rows x 16 columns of C x 64 parts of 64 k steps (4096 x 4128 x 4064)
    "sgemm": {"register": 64, "shared_memory": 0, "blocksize": 128, "solo_ptb_blks": 16,
              "ori_blks": 528384},
    # 10240 transforms of 256 points, a wavefront each; 2 KiB of LDS per wavefront
    "fft": {"register": 40, "shared_memory": 8192, "blocksize": 256, "solo_ptb_blks": 8,
            "ori_blks": 10240},
    # 26 x 26 x 2 regions of 8 x 8 x 8 lattice points (two wavefronts each) x 11 parts of 32 neighbour bins
    "cutcp": {"register": 48, "shared_memory": 0, "blocksize": 128, "solo_ptb_blks": 16,
              "ori_blks": 14872},
    # 2560000 blocks of 256 records; a stream that wants many workgroups in flight (4.0 TB/s with 8 a CU,
    # 4.95 with 32)
    "nn": {"register": 48, "shared_memory": 0, "blocksize": 256, "solo_ptb_blks": 32,
           "ori_blks": 2560000},
    # 256 x 2048 patches of 64 x 4 columns, 8 layers each; 24 streams of 256-byte pieces per patch: fewer
    # wavefronts in flight keep more of them in open memory pages (4.9 TB/s with 2 workgroups a CU, 3.9 with 8)
    "hot3d": {"register": 64, "shared_memory": 0, "blocksize": 256, "solo_ptb_blks": 2,
              "ori_blks": 524288},
    # 216000 boxes of 100 particles (a wavefront each) x 27 parts (the home box and its neighbour slots);
    # boxes on the faces have fewer neighbours: the more owner wavefronts, the evener their shares
    # (42.4 ms with 4 workgroups a CU, 35.8 with 32)
    "lava": {"register": 84, "shared_memory": 0, "blocksize": 256, "solo_ptb_blks": 32,
             "ori_blks": 5832000},
    # 200 windows of 256 columns (6 result columns each), a wavefront each
    "path": {"register": 64, "shared_memory": 0, "blocksize": 256, "solo_ptb_blks": 1,
             "ori_blks": 200},
    # 16384 blocks of 128 x 8 points x 4 parts of the unrolled x points
    "cp": {"register": 40, "shared_memory": 0, "blocksize": 128, "solo_ptb_blks": 16,
           "ori_blks": 65536},
}


def get_kernel_info(kernel_name, table=None):
    return (table or KERNEL_INFO)[kernel_name]


def fuse_kernel_info(kernel1_name, kernel2_name, table=None, budget=CDNA4_CU, max_copies=8,
                     reduce_gcd=True):
    """Candidates (blks_per_unit, n1, n2) for fusing kernel2 into kernel1's launch.

    kernel1 is the main kernel: it keeps exactly solo_ptb_blks * blocksize threads
    per SM/CU.  For every blocks-per-unit count and every number of kernel1 copies
    per block that gives that thread total, kernel2 copies are added while the
    thread, register and shared-memory totals fit the budget; (n1, n2) is reduced
    by its gcd into the block count.  Same enumeration order as the reference
    (fusion/code/data.py:48-69).  reduce_gcd=False lists the raw (blks, n1, n2)
    triples, which is what the candidate logs shipped with the reference
    (fusion/code/log.txt, mix_kernel_info.txt) were printed from; the file names
    under fusion/mix_kernel/ come from the reduced form.
    """
    table = table or KERNEL_INFO
    k1, k2 = table[kernel1_name], table[kernel2_name]
    k1_threads = k1["solo_ptb_blks"] * k1["blocksize"]
    candidates = []
    for blks in range(1, max_copies + 1):
        for n1 in range(1, max_copies + 1):
            if n1 * k1["blocksize"] * blks != k1_threads:
                continue
            for n2 in range(1, max_copies + 1):
                threads_ok = n2 * k2["blocksize"] * blks <= budget.thread_slots - k1_threads
                regs = (k1["register"] * n1 * blks * k1["blocksize"] +
                        k2["register"] * n2 * blks * k2["blocksize"])
                smem = k1["shared_memory"] * n1 * blks + k2["shared_memory"] * n2 * blks
                if threads_ok and regs <= budget.registers and smem <= budget.shared_memory:
                    g = gcd(n1, n2) if reduce_gcd else 1
                    cand = (blks * g, n1 // g, n2 // g)
                    if cand not in candidates:
                        candidates.append(cand)
    return candidates


def candidate_resources(kernel1_name, kernel2_name, cand, table=None):
    """(registers, shared memory, threads) per SM/CU of a candidate."""
    table = table or KERNEL_INFO
    k1, k2 = table[kernel1_name], table[kernel2_name]
    blks, n1, n2 = cand
    regs = blks * (n1 * k1["register"] * k1["blocksize"] + n2 * k2["register"] * k2["blocksize"])
    smem = blks * (n1 * k1["shared_memory"] + n2 * k2["shared_memory"])
    threads = blks * (n1 * k1["blocksize"] + n2 * k2["blocksize"])
    return regs, smem, threads


def pair_file_names(kernel1, kernel2, table=None, budget=CDNA4_CU):
    """File stems ``<k1>_<k2>_<r1>_<r2>`` the generator emits for a pair, both
    kernels taking the main role in turn (fusion/code/gen_mix.py:183-215)."""
    names = []
    done = []
    for blks, r1, r2 in fuse_kernel_info(kernel1, kernel2, table, budget):
        done.append((r1, r2))
        names.append(f"{kernel1}_{kernel2}_{r1}_{r2}")
    for blks, r2, r1 in fuse_kernel_info(kernel2, kernel1, table, budget):
        if (r1, r2) in done:
            continue
        names.append(f"{kernel1}_{kernel2}_{r1}_{r2}")
    return names
