"""Emit the text of fused ("mix") HIP kernels.

Counterpart of ``fusion/code/gen_mix.py`` of the reference
(``generate_mixed_kernel`` :16-76): one ``__global__`` whose parameter list is
the concatenation of both kernels' GPTB parameter lists, and whose body sends
each thread to one kernel's device-side role.  The reference splits by
``threadIdx.x`` thresholds and keeps each role's barriers apart with PTX named
barriers (``bar.sync id, n``).  gfx950 has one hardware barrier per workgroup,
so two forms are emitted:

* ``wg``   -- workgroup split: role = f(blockIdx); a group of ``a + b``
  consecutive XCD-slots holds ``a`` workgroups of the first kernel and ``b`` of
  the second (``tk::wg_split``).  Each role owns whole workgroups, so a role
  that needs a barrier uses the hardware one.
* ``wave`` -- wave split: every workgroup holds both roles, threads
  ``[0, t0)`` run the first kernel and ``[t0, t0 + t1)`` the second, the way the
  reference does; a role that needs a barrier uses an LDS arrival counter
  private to its waves until the other role's waves have ended, then the
  hardware barrier (``tk::RoleHandoverSync``).
"""
from kernel_code import ROLES, gptb_signature, signature


def _params_text(sig_a, sig_b):
    return ",\n    ".join(f"{t} {n}" for t, n in sig_a + sig_b)


def _void_unused(sig, body):
    """(void) casts for parameters the dispatcher body does not read."""
    import re
    return "".join(f"    (void){n};\n" for _, n in sig if not re.search(rf"\b{n}\b", body))


def mix_kernel_name(be, variant):
    return f"{be}_tzgemm_mix_{variant}"


def _stream_c(be):
    """Whether the GEMM role stores C with streaming stores in a kernel fused with ``be``: measured per
    pair (config 2 with the stencil 34.3 us without, 35.3 us with; the lbm pair 124 us without, 117 us
    with; no difference for mri-q and cp)."""
    return "false" if be == "stencil" else "true"


def generate_wg_split(be, tz_wgs, be_wgs, threads=256):
    """Workgroup-split fused kernel of ``be`` with tzgemm; tz_wgs : be_wgs per group."""
    variant = f"wg_{tz_wgs}_{be_wgs}"
    p_be, sig_be = signature(be, 0)
    p_tz, sig_tz = signature("tzgemm", 1)
    tz_call = ROLES["tzgemm"]["call"].format(p=p_tz, block="sp.role_block", blocks="sp.role_blocks",
                                             tid="(int)threadIdx.x", stages="TZ_STAGES_WG", stream_c=_stream_c(be))
    be_call = ROLES[be]["call"].format(p=p_be, block="sp.role_block", blocks="sp.role_blocks",
                                       tid="(int)threadIdx.x", threads=threads, waves=threads // 64, extra="")
    name = mix_kernel_name(be, variant)
    text = f"""// {be}-tzgemm  workgroup split  {tz_wgs} tzgemm : {be_wgs} {be} workgroups per group
extern "C" __global__ __launch_bounds__({threads}) void {name}(
    {_params_text(sig_be, sig_tz)})
{{
{_void_unused(sig_be + sig_tz, tz_call + be_call)}    __shared__ __align__(16) char tz_lds[TZ_LDS_BYTES_WG];
    const tk::WgSplit sp = tk::wg_split((int)blockIdx.x, (int)gridDim.x, {tz_wgs}, {be_wgs});
    if (sp.role == 0) {{
        tk::WorkgroupSync sync;
        {tz_call}
    }} else {{
        {be_call}
    }}
}}
"""
    meta = {"variant": variant, "symbol": name, "blocksize": threads,
            "group": tz_wgs + be_wgs, "tz_share": tz_wgs, "be_share": be_wgs, "kind": "wg"}
    return text, meta


# Template arguments of a role inside a wave-split kernel, where few best-effort waves share the CU
# with the GEMM: lbm takes two rows per wave to keep enough loads in flight, cutcp fetches every bin
# of atoms a bin ahead instead of waiting for it.
WAVE_SPLIT_EXTRA = {"lbm": "<2>", "cutcp": "<true>"}


def generate_wave_split(be, be_threads, tz_first=True, large=False):
    """Wave-split fused kernel: 256 tzgemm threads + be_threads of ``be`` per workgroup.

    large: the 512-thread form whose GEMM role takes 256 x 128 tiles (tzgemm_role_large_rot) for
    the shapes they divide (tz_large_fused_fits) and the 128 x 128 form for every other shape."""
    variant = f"wave_{be_threads}_large" if large else f"wave_{be_threads}"
    tz_threads = 256
    total = tz_threads + be_threads
    p_be, sig_be = signature(be, 0)
    p_tz, sig_tz = signature("tzgemm", 1)
    if tz_first:
        tz_lo, be_lo = 0, tz_threads
    else:
        be_lo, tz_lo = 0, be_threads
    tz_call = ROLES["tzgemm"]["call"].format(p=p_tz, block="(int)blockIdx.x",
                                             blocks=f"{p_tz}ptb_iter_block_step",
                                             tid=f"(int)threadIdx.x - {tz_lo}", stages="TZ_STAGES", stream_c=_stream_c(be))
    # few best-effort waves share the CU with the GEMM: see WAVE_SPLIT_EXTRA
    be_call = ROLES[be]["call"].format(p=p_be, block="be_block", blocks="be_blocks",
                                       tid=f"(int)threadIdx.x - {be_lo}", threads=be_threads,
                                       waves=be_threads // 64, extra=WAVE_SPLIT_EXTRA.get(be, ""))
    if large:
        if be_threads != 256:
            raise ValueError("the large-tile GEMM role needs the registers of a 512-thread workgroup")
        tz_call = (f"if (tz_large_fused_fits({p_tz}NORMAL_M, {p_tz}NORMAL_N, {p_tz}NORMAL_K))\n"
                   f"            tk::tzgemm_role_large_rot({p_tz}A, {p_tz}B, {p_tz}C, {p_tz}NORMAL_M, {p_tz}NORMAL_N, {p_tz}NORMAL_K, "
                   f"(int)blockIdx.x, {p_tz}ptb_iter_block_step, {p_tz}ptb_start_block_pos, {p_tz}ptb_end_block_pos, "
                   f"(int)threadIdx.x - {tz_lo}, tz_lds, {_stream_c(be)}, sync);\n"
                   f"        else\n            " + tz_call)
    tz_cond = (f"threadIdx.x < {tz_threads}" if tz_first else f"threadIdx.x >= {be_threads}")
    name = mix_kernel_name(be, variant)
    unused = _void_unused(sig_be + sig_tz, tz_call + be_call + f"{p_be}ptb_iter_block_step")
    text = f"""// {be}-tzgemm  wave split  {tz_threads} tzgemm threads + {be_threads} {be} threads per workgroup
extern "C" __global__ __launch_bounds__({total}) void {name}(
    {_params_text(sig_be, sig_tz)})
{{
{unused}    // One LDS object on purpose (ring + the arrival counter behind it): with two, the
    // compiler tags LDS accesses per object and then waits for every LDS-direct load in
    // flight before each read of the ring.
    __shared__ __align__(16) char tz_lds[TZ_LDS_BYTES + 16];
    unsigned *tz_arrivals = reinterpret_cast<unsigned *>(tz_lds + TZ_LDS_BYTES);
    if (threadIdx.x == 0) tk::RoleHandoverSync::init(tz_arrivals, {be_threads // 64});
    __syncthreads();   // the only barrier of all waves: before the roles part ways
    if ({tz_cond}) {{
        // One tzgemm wave per SIMD shares it with {be} waves: let the MFMA stream issue
        // whenever it is ready and the {be} waves fill the slots it leaves.
        __builtin_amdgcn_s_setprio(TK_GEMM_WAVE_PRIORITY);
        // role barrier: an arrival counter in LDS while {be} waves run, the hardware barrier once they have ended
        tk::RoleHandoverSync sync(tz_arrivals, {tz_threads // 64}, (int)threadIdx.x - {tz_lo}, &tk_spin_fail);
        {tz_call}
    }} else {{
        // A GEMM that leaves at least half of the workgroups without a tile: the {be} blocks go
        // to those workgroups only, where nothing competes with them, and the workgroups that
        // hold the latency-critical tiles run them undisturbed.
        const int launched = {p_be}ptb_iter_block_step;
        const int tz_busy = tk::tz_busy_workgroups({p_tz}NORMAL_M, {p_tz}NORMAL_N, {p_tz}NORMAL_K, launched,
                                                   {p_tz}ptb_start_block_pos, {p_tz}ptb_end_block_pos);
        const bool apart = 2 * tz_busy <= launched;
        const int be_block = apart ? (int)blockIdx.x - tz_busy : (int)blockIdx.x;
        const int be_blocks = apart ? launched - tz_busy : launched;
        if (be_block >= 0) {{
            {be_call}
        }}
        tk::role_wave_done(tz_arrivals);
    }}
}}
"""
    meta = {"variant": variant, "symbol": name, "blocksize": total, "group": 1,
            "tz_share": 1, "be_share": 1, "kind": "wave"}
    return text, meta


def be_pair_kernel_name(be1, be2, variant):
    return f"{be1}_{be2}_mix_{variant}"


def generate_be_pair(be1, be2, wgs1, wgs2, threads=256, order=False):
    """Fused kernel of two vector kernels (no tzgemm): workgroup split wgs1 : wgs2.

    Neither role uses LDS or a barrier, so workgroups of both kinds share a CU freely
    (``createMixKernel`` pairs of the reference, src/Creator.cu:341-816).  Parameter order:
    be1's GPTB list, then be2's; be1 < be2 alphabetically, as the reference names its pairs.

    ``wg_<a>_<b>``: the split fixes which kernel a workgroup serves -- a of every a + b
    workgroups run be1's blocks, the others be2's.  When the shorter kernel ends, its
    workgroups idle.

    ``ord_<a>_<b>`` (order=True): every workgroup serves both kernels, each kernel's blocks
    spread over all workgroups; the split only fixes the order -- a of every a + b workgroups
    start with be1 and go on to be2, the others the other way round.  While both kinds are at
    work a CU holds both kernels at once, and no workgroup ends before its share of both is
    done.
    """
    variant = f"{'ord' if order else 'wg'}_{wgs1}_{wgs2}"
    p1, sig1 = signature(be1, 0)
    p2, sig2 = signature(be2, 1)
    block, blocks = ("(int)blockIdx.x", "(int)gridDim.x") if order else ("sp.role_block", "sp.role_blocks")
    call1 = ROLES[be1]["call"].format(p=p1, block=block, blocks=blocks, tid="(int)threadIdx.x", threads=threads,
                                      waves=threads // 64, extra="")
    call2 = ROLES[be2]["call"].format(p=p2, block=block, blocks=blocks, tid="(int)threadIdx.x", threads=threads,
                                      waves=threads // 64, extra="")
    name = be_pair_kernel_name(be1, be2, variant)
    if order:
        title = f"order split  {wgs1} of {wgs1 + wgs2} workgroups start with {be1}, the others with {be2}"
        body = f"""    for (int phase = 0; phase < 2; ++phase) {{
        if ((sp.role ^ phase) == 0) {{
            {call1}
        }} else {{
            {call2}
        }}
    }}"""
    else:
        title = f"workgroup split  {wgs1} {be1} : {wgs2} {be2} workgroups per group"
        body = f"""    if (sp.role == 0) {{
        {call1}
    }} else {{
        {call2}
    }}"""
    text = f"""// {be1}-{be2}  {title}
extern "C" __global__ __launch_bounds__({threads}) void {name}(
    {_params_text(sig1, sig2)})
{{
{_void_unused(sig1 + sig2, call1 + call2)}    const tk::WgSplit sp = tk::wg_split((int)blockIdx.x, (int)gridDim.x, {wgs1}, {wgs2});
{body}
}}
"""
    meta = {"variant": variant, "symbol": name, "blocksize": threads, "group": wgs1 + wgs2,
            "share1": wgs1, "share2": wgs2, "kind": "wg"}
    return text, meta


# wavefronts a GPTB launch of a role that sizes its LDS by them may have (__launch_bounds__(256))
GPTB_MAX_WAVES = 4


def generate_gptb(name):
    """The plain GPTB kernel of one role (``src/gptb_kernel/<name>_kernel.cu`` of the reference): the
    launch's workgroups are the role's persistent workgroups, ``thread_base`` shifts the thread index
    (src/GPTBKernel.h:30-61).  Returns (text, symbol)."""
    role = ROLES[name]
    sig = gptb_signature(name)
    call = role["call"].format(p="", block="(int)blockIdx.x", blocks="ptb_iter_block_step",
                               tid="(int)threadIdx.x - thread_base", threads="(int)blockDim.x", waves=GPTB_MAX_WAVES,
                               extra="",
                               stages="TZ_STAGES", stream_c="true")
    symbol = role["gptb"]["symbol"]
    attributes = role["gptb"]["attributes"] + " " if role["gptb"]["attributes"] else ""
    setup = ""
    if name == "tzgemm":
        setup = ("    __shared__ __align__(16) char tz_lds[TZ_LDS_BYTES];\n"
                 "    tk::WorkgroupSync sync;\n")
    text = f"""// Generated by fusion/code/gen_run.py -- do not edit.
// GPTB form of {name} ({role["gptb"]["cite"]}): block positions [ptb_start_block_pos,
// ptb_end_block_pos) served by the ptb_iter_block_step workgroups of the launch.
extern "C" __global__ {attributes}void {symbol}(
    {_params_text(sig, [])})
{{
{_void_unused(sig, call)}{setup}    {call}
}}
"""
    return text, symbol


def generate_pair(be, candidates):
    """All fused kernels of one (be, tzgemm) pair: yields (text, meta)."""
    for cand in candidates:
        if cand[0] == "wg":
            yield generate_wg_split(be, cand[1], cand[2])
        elif cand[0] == "wave":
            yield generate_wave_split(be, cand[1])
        elif cand[0] == "wave_large":
            yield generate_wave_split(be, cand[1], large=True)
        else:
            raise ValueError(cand)
