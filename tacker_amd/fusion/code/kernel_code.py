"""Role descriptions the generator stitches together.

Each entry plays the part of one ``<kernel>_code.py`` of the reference
(fusion/code/cp_code.py, cutcp_code.py, fft_code.py, lbm_code.py, mriq_code.py, mrif_code.py, sgemm_code.py, stencil_code.py and the
truncated tzgemm_code.py; the Rodinia kernels nn, hot3d, lava and path have no such file there, their fused
kernels are checked in under src/mix_kernel): the kernel's parameter list in reference order and
how to call its device-side role.  The role bodies themselves live in
``csrc/kernels/*_role.h``; the generator emits dispatchers around them, the way
the reference's generated ``__global__`` functions call ``<a>_<b>_<k><i>()``
device functions.

``params``   -- (C type, name) in the order of the reference kernel's signature,
               without the 10-int GPTB trailer.
``gptb``     -- the plain GPTB kernel of the role: its symbol (the reference's names,
               src/main.cu:108-125: ``g_general_ptb_`` for mriq and cp), attributes in front
               of ``void`` and the reference file that holds its counterpart.
``call``     -- format string of the role call; ``{p}`` is the parameter prefix,
               ``{block}``, ``{blocks}`` the role-local persistent-workgroup id
               and count, ``{tid}`` the role-local thread id, ``{threads}`` the
               role's thread count, ``{waves}`` that count in wavefronts (a compile-time
               constant: it sizes the role's LDS), ``{extra}`` role-specific trailing arguments.
"""

GPTB_DIMS = ["grid_dimension_x", "grid_dimension_y", "grid_dimension_z",
             "block_dimension_x", "block_dimension_y", "block_dimension_z"]
GPTB_RANGE = ["ptb_start_block_pos", "ptb_iter_block_step", "ptb_end_block_pos"]

ROLES = {
    "tzgemm": {
        "gptb": {"symbol": "general_ptb_tzgemm", "cite": "src/gptb_kernel/tzgemm_kernel.cu:430-448",
                 "attributes": "__launch_bounds__(TZ_THREADS) __attribute__((amdgpu_waves_per_eu(1, 1)))"},
        "params": [("_Float16*", "A"), ("_Float16*", "B"), ("float*", "C"),
                   ("int", "NORMAL_M"), ("int", "NORMAL_N"), ("int", "NORMAL_K")],
        "needs_sync": True,
        "lds_bytes": "TZ_LDS_BYTES",
        "call": ("tk::tzgemm_role<{stages}, {stream_c}>({p}A, {p}B, {p}C, {p}NORMAL_M, {p}NORMAL_N, {p}NORMAL_K, "
                 "tk::tz_workspace_of({p}C, {p}NORMAL_M, {p}NORMAL_N, {p}NORMAL_K), {block}, {blocks}, {p}ptb_start_block_pos, {p}ptb_end_block_pos, {tid}, "
                 "tz_lds, sync);"),
    },
    "stencil": {
        "gptb": {"symbol": "general_ptb_stencil", "cite": "src/gptb_kernel/stencil_kernel.cu:3-105",
                 "attributes": "__launch_bounds__(256)"},
        "params": [("float", "c0"), ("float", "c1"), ("float*", "A0"), ("float*", "Anext"),
                   ("int", "nx"), ("int", "ny"), ("int", "nz")],
        "needs_sync": False,
        "call": ("tk::stencil_role({p}c0, {p}c1, {p}A0, {p}Anext, {p}nx, {p}ny, {p}nz, "
                 "{p}grid_dimension_x, {p}grid_dimension_y, {p}grid_dimension_z, {block}, {blocks}, "
                 "{p}ptb_start_block_pos, {p}ptb_end_block_pos, {tid}, {threads});"),
    },
    "lbm": {
        "gptb": {"symbol": "general_ptb_lbm", "cite": "src/gptb_kernel/lbm_kernel.cu:3-178", "attributes": ""},
        "params": [("float*", "srcGrid"), ("float*", "dstGrid")],
        "needs_sync": False,
        "call": ("tk::lbm_role{extra}({p}srcGrid, {p}dstGrid, {p}grid_dimension_x, {p}grid_dimension_y, "
                 "{p}block_dimension_x, {block}, {blocks}, {p}ptb_start_block_pos, "
                 "{p}ptb_end_block_pos, {tid}, {threads});"),
    },
    "mriq": {
        "gptb": {"symbol": "g_general_ptb_mriq", "cite": "src/gptb_kernel/mriq_kernel.cu:3-70", "attributes": ""},
        "params": [("int", "numK"), ("int", "kGlobalIndex"), ("float*", "x"), ("float*", "y"),
                   ("float*", "z"), ("float*", "Qr"), ("float*", "Qi")],
        "needs_sync": False,
        "call": ("tk::mriq_role({p}numK, {p}x, {p}y, {p}z, {p}Qr, {p}Qi, {p}grid_dimension_x, "
                 "{p}grid_dimension_y, {block}, {blocks}, {p}ptb_start_block_pos, {p}ptb_end_block_pos, {tid}, "
                 "{threads});"),
    },
    "mrif": {
        "gptb": {"symbol": "general_ptb_mrif", "cite": "src/gptb_kernel/mrif_kernel.cu:6-93", "attributes": ""},
        "params": [("int", "numK"), ("int", "kGlobalIndex"), ("float*", "x"), ("float*", "y"),
                   ("float*", "z"), ("float*", "outR"), ("float*", "outI")],
        "needs_sync": False,
        "call": ("tk::mrif_role({p}numK, {p}x, {p}y, {p}z, {p}outR, {p}outI, {p}grid_dimension_x, "
                 "{p}grid_dimension_y, {block}, {blocks}, {p}ptb_start_block_pos, {p}ptb_end_block_pos, {tid}, "
                 "{threads});"),
    },
    "sgemm": {
        "gptb": {"symbol": "general_ptb_sgemm", "cite": "src/gptb_kernel/sgemm_kernel.cu:3-66",
                 "attributes": "__launch_bounds__(256)"},
        "params": [("float*", "A"), ("float*", "B"), ("float*", "C"),
                   ("int", "NORMAL_M"), ("int", "NORMAL_N"), ("int", "NORMAL_K")],
        "needs_sync": False,
        "call": ("tk::sgemm_role({p}A, {p}B, {p}C, {p}NORMAL_M, {p}NORMAL_N, {p}NORMAL_K, {p}grid_dimension_x, "
                 "{p}grid_dimension_y, {p}grid_dimension_z, {block}, {blocks}, {p}ptb_start_block_pos, "
                 "{p}ptb_end_block_pos, {tid}, {threads});"),
    },
    "fft": {
        "gptb": {"symbol": "g_general_ptb_fft", "cite": "src/gptb_kernel/fft_kernel.cu:39-75",
                 "attributes": "__launch_bounds__(256)"},
        "params": [("float*", "data")],
        "needs_sync": False,
        "call": ("tk::fft_role<{waves}>({p}data, {p}grid_dimension_x, {block}, {blocks}, {p}ptb_start_block_pos, "
                 "{p}ptb_end_block_pos, {tid}, {threads});"),
    },
    "cutcp": {
        "gptb": {"symbol": "general_ptb_cutcp", "cite": "src/gptb_kernel/cutcp_kernel.cu:12-183", "attributes": ""},
        "params": [("int", "binDim_x"), ("int", "binDim_y"), ("float*", "binZeroAddr"), ("float", "h"),
                   ("float", "cutoff2"), ("float", "inv_cutoff2"), ("float*", "regionZeroAddr"),
                   ("int", "zRegionIndex_t")],
        "needs_sync": False,
        "call": ("tk::cutcp_role{extra}({p}binDim_x, {p}binDim_y, {p}binZeroAddr, {p}h, {p}cutoff2, {p}inv_cutoff2, "
                 "{p}regionZeroAddr, {p}grid_dimension_x, {p}grid_dimension_y, {p}grid_dimension_z, {block}, {blocks}, "
                 "{p}ptb_start_block_pos, {p}ptb_end_block_pos, {tid}, {threads});"),
    },
    "nn": {
        "gptb": {"symbol": "general_ptb_nn", "cite": "src/gptb_kernel/nn_kernel.cu:3-23",
                 "attributes": "__launch_bounds__(256)"},
        "params": [("LatLong*", "d_locations"), ("float*", "d_distances"), ("int", "numRecords"),
                   ("float", "lat"), ("float", "lng")],
        "needs_sync": False,
        "call": ("tk::nn_role({p}d_locations, {p}d_distances, {p}numRecords, {p}lat, {p}lng, {p}grid_dimension_x, "
                 "{p}grid_dimension_y, {p}block_dimension_x, {block}, {blocks}, {p}ptb_start_block_pos, "
                 "{p}ptb_end_block_pos, {tid}, {threads});"),
    },
    "hot3d": {
        "gptb": {"symbol": "general_ptb_hot3d", "cite": "src/gptb_kernel/hot3d_kernel.cu:3-62",
                 "attributes": "__launch_bounds__(256)"},
        "params": [("float*", "p"), ("float*", "tIn"), ("float*", "tOut"), ("float", "sdc"),
                   ("int", "nx"), ("int", "ny"), ("int", "nz"), ("float", "ce"), ("float", "cw"),
                   ("float", "cn"), ("float", "cs"), ("float", "ct"), ("float", "cb"), ("float", "cc")],
        "needs_sync": False,
        "call": ("tk::hot3d_role({p}p, {p}tIn, {p}tOut, {p}sdc, {p}nx, {p}ny, {p}nz, {p}ce, {p}cw, {p}cn, {p}cs, "
                 "{p}ct, {p}cb, {p}cc, {p}grid_dimension_x, {p}grid_dimension_y, {p}block_dimension_x, "
                 "{p}block_dimension_y, {block}, {blocks}, {p}ptb_start_block_pos, {p}ptb_end_block_pos, {tid}, "
                 "{threads});"),
    },
    "lava": {
        "gptb": {"symbol": "general_ptb_lava", "cite": "src/gptb_kernel/lava_kernel.cu:3-140",
                 "attributes": "__launch_bounds__(256)"},
        "params": [("par_str", "d_par_gpu"), ("dim_str", "d_dim_gpu"), ("box_str*", "d_box_gpu"),
                   ("FOUR_VECTOR*", "d_rv_gpu"), ("float*", "d_qv_gpu"), ("FOUR_VECTOR*", "d_fv_gpu")],
        "needs_sync": False,
        "call": ("tk::lava_role({p}d_par_gpu, {p}d_dim_gpu, {p}d_box_gpu, {p}d_rv_gpu, {p}d_qv_gpu, {p}d_fv_gpu, "
                 "{p}grid_dimension_x, {block}, {blocks}, {p}ptb_start_block_pos, {p}ptb_end_block_pos, {tid}, "
                 "{threads});"),
    },
    "path": {
        "gptb": {"symbol": "general_ptb_path", "cite": "src/gptb_kernel/path_kernel.cu:3-93",
                 "attributes": "__launch_bounds__(256)"},
        "params": [("int", "iteration"), ("int*", "gpuWall"), ("int*", "gpuSrc"), ("int*", "gpuResults"),
                   ("int", "cols"), ("int", "rows"), ("int", "startStep"), ("int", "border")],
        "needs_sync": False,
        "call": ("tk::path_role({p}iteration, {p}gpuWall, {p}gpuSrc, {p}gpuResults, {p}cols, {p}startStep, "
                 "{p}border, {block}, {blocks}, {p}ptb_start_block_pos, {p}ptb_end_block_pos, {tid}, {threads});"),
    },
    "cp": {
        "gptb": {"symbol": "g_general_ptb_cp", "cite": "src/gptb_kernel/cp_kernel.cu:8-96", "attributes": ""},
        "params": [("int", "numatoms"), ("float", "gridspacing"), ("float*", "energygrid")],
        "needs_sync": False,
        "call": ("tk::cp_role({p}numatoms, {p}gridspacing, {p}energygrid, {p}grid_dimension_x, "
                 "{p}grid_dimension_y, {p}grid_dimension_z, {block}, {blocks}, {p}ptb_start_block_pos, "
                 "{p}ptb_end_block_pos, {tid}, {threads});"),
    },
}


def signature(name, index):
    """Parameter list of role ``name`` as the index-th kernel of a fused launch:
    ori params, 6 GPTB dims, start/step/end -- the concatenation MixKernel builds
    (src/MixKernel.h:55-73 of the reference); no thread_base (it is baked in)."""
    prefix = f"{name}{index}_"
    out = [(t, prefix + n) for t, n in ROLES[name]["params"]]
    out += [("int", prefix + n) for n in GPTB_DIMS + GPTB_RANGE]
    return prefix, out


def gptb_signature(name):
    """Parameter list of the plain GPTB kernel of role ``name``: ori params, 6 GPTB dims,
    start/step/end, thread_base (src/GPTBKernel.h:30-61 of the reference appends them in this order)."""
    out = list(ROLES[name]["params"])
    out += [("int", n) for n in GPTB_DIMS + GPTB_RANGE + ["thread_base"]]
    return out
