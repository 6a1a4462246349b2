"""Python face of libtacker_amd.so (ctypes over the C-ABI of include/tacker_amd.h).

PyTorch is used by callers only as the owner of device memory and streams; every
compute call here goes through the C entry points, which launch the hand-written
gfx950 kernels.  There is no fallback: if the library is missing or a call fails,
an exception is raised.

    import tacker_amd as ta
    ta.init()                                  # tacker_init(0, builtin kinfo)
    ta.gptb_tzgemm(A, B, C)                    # torch tensors on cuda:0
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libtacker_amd.so")
FAKE_LIB_PATH = os.path.join(_HERE, "lib", "libtacker_host_fake.so")
# the device code alone, as code objects for tacker_register_module
CODE_OBJECT_PATH = os.path.join(_HERE, "lib", "tacker_kernels.hsaco")
CODE_OBJECT_LARGE_PATH = os.path.join(_HERE, "lib", "tacker_kernels_large.hsaco")
KINFO_PATH = os.path.join(_HERE, "config", "kinfo-gfx950.json")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "tacker_amd.h")

JSON_NOT_FOUND = -32767
ALPHA = 1.1


class TackerError(RuntimeError):
    pass


def _declare(lib):
    vp, i, f, cp = C.c_void_p, C.c_int, C.c_float, C.c_char_p
    lib.tacker_init.argtypes = [i, cp]
    lib.tacker_last_error.restype = cp
    lib.tkGetErrorString.restype = cp
    lib.tkGetErrorString.argtypes = [i]
    lib.tkGetCuCount.argtypes = [C.POINTER(i)]
    lib.tkGetDeviceName.argtypes = [C.c_char_p, C.c_size_t]
    lib.tacker_tzgemm_grid_dim.argtypes = [i, i, i, C.POINTER(i)]
    lib.tacker_gptb_tzgemm.argtypes = [vp, vp, vp, i, i, i, i, i, i, vp]
    lib.tacker_gptb_tzgemm_static_scratch.argtypes = [vp, vp, vp, i, i, i, i, i, i, vp]
    lib.tacker_ori_stencil.argtypes = [f, f, vp, vp, i, i, i, vp]
    lib.tacker_stencil_blocks.argtypes = [i, i, i]
    lib.tacker_gptb_stencil.argtypes = [f, f, vp, vp, i, i, i, i, i, i, i, vp]
    lib.tacker_ori_lbm.argtypes = [vp, vp, i, i, i, vp]
    lib.tacker_gptb_lbm.argtypes = [vp, vp, i, i, i, i, i, i, i, vp]
    lib.tacker_mriq_phimag.argtypes = [vp, vp, vp, i, vp]
    lib.tacker_mriq_set_kvalues.argtypes = [vp, i]
    lib.tacker_mriq_blocks.argtypes = [i, i]
    lib.tacker_cp_blocks.argtypes = [i, i]
    lib.tacker_cp_inv_sqrt_selftest.argtypes = [C.c_uint, C.c_uint, C.POINTER(C.c_ulonglong)]
    lib.tacker_ori_mriq.argtypes = [i, vp, vp, vp, vp, vp, i, vp]
    lib.tacker_gptb_mriq.argtypes = [i, vp, vp, vp, vp, vp, i, i, i, i, i, vp]
    lib.tacker_cp_set_atoms.argtypes = [vp, i, f]
    lib.tacker_cp_initatoms.argtypes = [vp, i, C.c_uint, C.c_uint, C.c_uint, f]
    lib.tacker_ori_cp.argtypes = [i, f, vp, i, i, vp]
    lib.tacker_gptb_cp.argtypes = [i, f, vp, i, i, i, i, i, i, vp]
    gemm = [vp, vp, vp, i, i, i, i, i, cp, i, i, vp]
    lib.tacker_mix_tzgemm_stencil.argtypes = [f, f, vp, vp, i, i, i, i, i] + gemm
    lib.tacker_mix_tzgemm_lbm.argtypes = [vp, vp, i, i, i, i, i] + gemm
    lib.tacker_mix_tzgemm_mriq.argtypes = [i, vp, vp, vp, vp, vp, i, i, i] + gemm
    lib.tacker_mrif_rhophi.argtypes = [i, vp, vp, vp, vp, vp, vp, vp]
    lib.tacker_mrif_set_kvalues.argtypes = [vp, i]
    lib.tacker_mrif_blocks.argtypes = [i, i]
    lib.tacker_ori_mrif.argtypes = [i, vp, vp, vp, vp, vp, i, vp]
    lib.tacker_gptb_mrif.argtypes = [i, vp, vp, vp, vp, vp, i, i, i, i, i, vp]
    lib.tacker_mix_tzgemm_mrif.argtypes = [i, vp, vp, vp, vp, vp, i, i, i] + gemm
    lib.tacker_sgemm_blocks.argtypes = [i, i, i]
    lib.tacker_ori_sgemm.argtypes = [vp, vp, vp, i, i, i, vp]
    lib.tacker_gptb_sgemm.argtypes = [vp, vp, vp, i, i, i, i, i, i, i, vp]
    lib.tacker_mix_tzgemm_sgemm.argtypes = [vp, vp, vp, i, i, i, i, i] + gemm
    cut = [i, i, vp, f, f, f, vp, i, i, i]
    lib.tacker_cutcp_prepare_input.argtypes = [vp, i, vp, i, i, i, f, f, vp, vp, vp, vp, vp, vp]
    lib.tacker_cutcp_set_neighbours.argtypes = [vp, i]
    lib.tacker_cutcp_blocks.argtypes = [i, i, i]
    lib.tacker_ori_cutcp.argtypes = cut + [vp]
    lib.tacker_gptb_cutcp.argtypes = cut + [i, i, i, i, vp]
    lib.tacker_mix_tzgemm_cutcp.argtypes = cut + [i, i] + gemm
    lib.tacker_ori_fft.argtypes = [vp, i, vp]
    lib.tacker_gptb_fft.argtypes = [vp, i, i, i, i, i, vp]
    lib.tacker_mix_tzgemm_fft.argtypes = [vp, i, i, i] + gemm
    lib.tacker_mix_tzgemm_cp.argtypes = [i, f, vp, i, i, i, i] + gemm
    lib.tacker_nn_blocks.argtypes = [i]
    lib.tacker_ori_nn.argtypes = [vp, vp, i, f, f, vp]
    lib.tacker_gptb_nn.argtypes = [vp, vp, i, f, f, i, i, i, i, vp]
    lib.tacker_mix_tzgemm_nn.argtypes = [vp, vp, i, f, f, i, i] + gemm
    lib.tacker_hot3d_coefficients.argtypes = [i, i, i, vp]
    lib.tacker_ori_hot3d.argtypes = [vp, vp, vp, i, i, i, vp]
    lib.tacker_gptb_hot3d.argtypes = [vp, vp, vp, i, i, i, i, i, i, i, vp]
    lib.tacker_mix_tzgemm_hot3d.argtypes = [vp, vp, vp, i, i, i, i, i] + gemm
    lib.tacker_lava_blocks.argtypes = [i]
    lib.tacker_lava_boxes.argtypes = [i, vp, C.c_size_t]
    lib.tacker_ori_lava.argtypes = [f, i, vp, vp, vp, vp]
    lib.tacker_gptb_lava.argtypes = [f, i, vp, vp, vp, i, i, i, i, vp]
    lib.tacker_mix_tzgemm_lava.argtypes = [f, i, vp, vp, vp, i, i] + gemm
    lib.tacker_path_blocks.argtypes = [i, i]
    lib.tacker_ori_path.argtypes = [i, vp, vp, vp, i, i, i, vp]
    lib.tacker_gptb_path.argtypes = [i, vp, vp, vp, i, i, i, i, i, i, i, vp]
    lib.tacker_mix_tzgemm_path.argtypes = [i, vp, vp, vp, i, i, i, i, i] + gemm
    lib.tacker_im2col.argtypes = [vp] + [i] * 11 + [vp, vp]
    lib.tacker_convert_fp32_to_fp16.argtypes = [vp, vp, i, vp]
    lib.tacker_mnk_from_conv_args.argtypes = [C.POINTER(i), C.POINTER(i)]
    lib.tacker_get_kernel_info.argtypes = [cp, cp]
    lib.tacker_fget_kernel_info.argtypes = [cp, cp]
    lib.tacker_fget_kernel_info.restype = f
    for name in ("tacker_create_kernel", "tacker_ori_stencil_create", "tacker_ori_lbm_create",
                 "tacker_ori_mriq_create", "tacker_ori_mrif_create", "tacker_ori_cp_create", "tacker_ori_tzgemm_create",
                 "tacker_ori_sgemm_create", "tacker_ori_fft_create", "tacker_ori_cutcp_create",
                 "tacker_ori_nn_create", "tacker_ori_hot3d_create", "tacker_ori_path_create", "tacker_ori_lava_create",
                 "tacker_gptb_create", "tacker_mix_create", "tacker_be_pair_create",
                 "tacker_create_mix_kernel"):
        getattr(lib, name).restype = vp
    lib.tacker_create_kernel.argtypes = [cp]
    lib.tacker_ori_stencil_create.argtypes = [f, f, vp, vp, i, i, i]
    lib.tacker_ori_lbm_create.argtypes = [vp, vp, i, i, i]
    lib.tacker_ori_mriq_create.argtypes = [i, vp, vp, vp, vp, vp, i]
    lib.tacker_ori_mrif_create.argtypes = [i, vp, vp, vp, vp, vp, i]
    lib.tacker_ori_sgemm_create.argtypes = [vp, vp, vp, i, i, i]
    lib.tacker_ori_fft_create.argtypes = [vp, i]
    lib.tacker_ori_nn_create.argtypes = [vp, vp, i, f, f]
    lib.tacker_ori_hot3d_create.argtypes = [vp, vp, vp, i, i, i]
    lib.tacker_ori_path_create.argtypes = [i, vp, vp, vp, i, i, i]
    lib.tacker_ori_lava_create.argtypes = [f, i, vp, vp, vp]
    lib.tacker_ori_cutcp_create.argtypes = cut
    lib.tacker_ori_cp_create.argtypes = [i, f, vp, i, i]
    lib.tacker_ori_tzgemm_create.argtypes = [vp, vp, vp, i, i, i]
    lib.tacker_gptb_create.argtypes = [vp, i, i, i, i]
    lib.tacker_gptb_set_range.argtypes = [vp, i, i]
    lib.tacker_mix_create.argtypes = [vp, vp, i, i, i, i, cp, i, i]
    lib.tacker_mix_set_range.argtypes = [vp, i, i, i, i]
    lib.tacker_be_pair_create.argtypes = [vp, vp, i, i, i, i, cp, i]
    lib.tacker_create_mix_kernel.argtypes = [cp]
    lib.tacker_kernel_execute.argtypes = [vp, vp]
    lib.tacker_kernel_swap_buffers.argtypes = [vp]
    lib.tacker_kernel_info.argtypes = [vp, C.POINTER(i)]
    lib.tacker_kernel_param.argtypes = [vp, i, vp, i]
    lib.tacker_register_module.argtypes = [C.c_char_p, C.c_char_p]
    lib.tacker_module_has_function.argtypes = [C.c_char_p, C.c_char_p]
    lib.tacker_kernel_use_module.argtypes = [vp, C.c_char_p, C.c_char_p]
    lib.tacker_mix_cublas_sgemm.argtypes = [C.POINTER(i), vp, i, i, vp]
    lib.tacker_mix_cudnn_convolution_forward.argtypes = [C.POINTER(i), vp, i, i, vp]
    lib.tacker_kernel_destroy.argtypes = [vp]
    lib.tacker_spin_fail_flag.argtypes = [C.POINTER(i)]
    lib.tacker_float_to_half_bits.argtypes = [f]
    lib.tacker_float_to_half_bits.restype = C.c_uint16
    lib.tacker_tzgemm_workspace_bytes.restype = C.c_longlong
    lib.tacker_rng_uniform.argtypes = [C.c_uint64, f, f, vp, C.c_size_t]
    lib.tacker_task_create.restype = vp
    lib.tacker_task_create.argtypes = [cp, i, i]
    lib.tacker_task_destroy.argtypes = [vp]
    lib.tacker_task_execute.argtypes = [vp, vp]
    lib.tacker_task_kernel_count.argtypes = [vp]
    lib.tacker_task_kernel_info.argtypes = [vp, i, C.c_char_p, i, C.POINTER(i), C.POINTER(i), C.POINTER(i)]
    lib.tacker_task_activation.argtypes = [vp, i, C.POINTER(vp), C.POINTER(i)]
    lib.tacker_task_conv_params.argtypes = [vp, i, C.POINTER(vp), C.POINTER(vp), C.POINTER(i)]
    lib.tkMemcpy.argtypes = [vp, vp, C.c_size_t, i]
    lib.tkMemset.argtypes = [vp, i, C.c_size_t]
    lib.tacker_task_logits.argtypes = [vp, C.POINTER(vp), C.POINTER(C.c_long), C.POINTER(i)]
    lib.tacker_task_input.argtypes = [vp, C.POINTER(vp), C.POINTER(i)]
    lib.tacker_task_stage_input.argtypes = [vp]
    lib.tacker_task_capture.argtypes = [vp, vp, C.POINTER(vp)]
    lib.tkAllocationCalls.argtypes = [C.POINTER(C.c_longlong), C.POINTER(C.c_longlong)]
    lib.tkStreamCreate.argtypes = [C.POINTER(vp)]
    lib.tkStreamDestroy.argtypes = [vp]
    lib.tkStreamSynchronize.argtypes = [vp]
    lib.tkStreamBeginCapture.argtypes = [vp]
    lib.tkStreamEndCapture.argtypes = [vp, C.POINTER(vp)]
    lib.tkGraphLaunch.argtypes = [vp, vp]
    lib.tkGraphExecDestroy.argtypes = [vp]
    lib.tacker_task_manager_create.restype = vp
    lib.tacker_task_manager_create.argtypes = [vp, cp, cp]
    lib.tacker_task_manager_destroy.argtypes = [vp]
    lib.tacker_task_manager_configure.argtypes = [vp, f, f, i, i, i, i]
    lib.tacker_task_manager_run.argtypes = [vp, i, vp, i]
    lib.tacker_task_manager_report.argtypes = [vp, C.POINTER(f)]
    lib.tacker_task_manager_latencies.argtypes = [vp, i, C.POINTER(f), i]
    lib.tacker_task_manager_set_fusion_strikes.argtypes = [vp, i]
    lib.tacker_task_manager_fusion_disabled.argtypes = [vp]
    lib.tacker_task_manager_set_calibration.argtypes = [vp, i, f]
    lib.tacker_task_manager_set_end_to_end.argtypes = [vp, i]
    lib.tacker_task_manager_calibrated_blocks.argtypes = [vp, vp, i]
    lib.tacker_task_manager_set_calibration_budget.argtypes = [vp, f, i]
    lib.tacker_task_manager_set_calibration_variants.argtypes = [vp, cp]
    lib.tacker_task_manager_calibrated_variant.argtypes = [vp, i, cp, i]
    lib.tacker_task_manager_be_mix_ms.argtypes = [vp]
    lib.tacker_task_manager_be_mix_ms.restype = f
    lib.tacker_qos_block_ratio.argtypes = [cp, i]
    lib.tacker_qos_block_ratio.restype = f
    lib.tacker_qos_whole_kernel_gain.argtypes = [cp]
    lib.tacker_qos_whole_kernel_gain.restype = f
    lib.tacker_qos_colocated_blocks.argtypes = [i, cp, i, i, i]
    lib.tacker_qos_must_run_solo.argtypes = [f, f, f, f]
    lib.tacker_qos_account.argtypes = [i, f, f, f, i, i, C.POINTER(f)]
    return lib


def load_library(path=LIB_PATH):
    """dlopen a build of the host runtime (the HIP one by default)."""
    if not os.path.exists(path):
        raise TackerError(f"{path} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                          "(or make -C tacker_amd/csrc) first; there is no fallback path")
    return _declare(C.CDLL(path))


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = load_library()
    return _lib


def check(rc, what="tacker call"):
    if rc != 0:
        raise TackerError(f"{what} failed ({rc}): {lib().tacker_last_error().decode()}")


def init(device=0, kinfo=None):
    """tacker_init: device, kernel registry, kinfo table (None = built-in)."""
    check(lib().tacker_init(device, kinfo.encode() if kinfo else None), "tacker_init")


def cu_count():
    n = C.c_int()
    check(lib().tkGetCuCount(C.byref(n)), "tkGetCuCount")
    return n.value


def device_name():
    buf = C.create_string_buffer(256)
    check(lib().tkGetDeviceName(buf, 256), "tkGetDeviceName")
    return buf.value.decode()


def tzgemm_grid_dim(m, n, k):
    out = (C.c_int * 4)()
    lib().tacker_tzgemm_grid_dim(m, n, k, out)
    return list(out)


def tzgemm_parts(m, n, k):
    """Workgroups that share the reduction of one tile of this shape (1 for most shapes)."""
    return int(lib().tacker_tzgemm_parts(m, n, k))


def tzgemm_workspace_bytes(m, n, k):
    return int(lib().tacker_tzgemm_workspace_bytes(m, n, k))


def tzgemm_release_workspaces():
    check(lib().tacker_tzgemm_release_workspaces(), "tzgemm_release_workspaces")


def get_kernel_info(kernel, key):
    return lib().tacker_get_kernel_info(kernel.encode(), key.encode())


def fget_kernel_info(kernel, key):
    return lib().tacker_fget_kernel_info(kernel.encode(), key.encode())


def _ptr(t):
    """Device pointer of a torch tensor (must be contiguous and on the GPU)."""
    if t is None:
        return None
    if not t.is_cuda or not t.is_contiguous():
        raise TackerError("tensors must be contiguous CUDA/HIP tensors")
    return t.data_ptr()


def _stream(stream):
    if stream is None:
        import torch
        return torch.cuda.current_stream().cuda_stream
    return getattr(stream, "cuda_stream", stream)


def _v(variant):
    return variant.encode() if variant else None


# ----------------------------------------------------------------------------- one-shot calls
def gptb_tzgemm(A, B, Cm, tile_start=0, tile_end=None, launch_grid=0, stream=None):
    M, K = A.shape
    N = B.shape[0]
    if tile_end is None:
        tile_end = (M // 64) * (N // 64)
    check(lib().tacker_gptb_tzgemm(_ptr(A), _ptr(B), _ptr(Cm), M, N, K, tile_start, tile_end,
                                   launch_grid, _stream(stream)), "tacker_gptb_tzgemm")


def gptb_tzgemm_static_scratch(A, B, Cm, tile_start=0, tile_end=None, launch_grid=0, stream=None):
    """gptb_tzgemm that allocates nothing: its workspace is the library's static device array"""
    M, K = A.shape
    N = B.shape[0]
    if tile_end is None:
        tile_end = (M // 64) * (N // 64)
    check(lib().tacker_gptb_tzgemm_static_scratch(_ptr(A), _ptr(B), _ptr(Cm), M, N, K, tile_start, tile_end,
                                                  launch_grid, _stream(stream)), "tacker_gptb_tzgemm_static_scratch")


def stencil_blocks(nx, ny, nz=None):
    """block positions of the GPTB form: blocks of 64 x 4 columns, times (when nz is given) the runs of
    8 centre planes a block column is cut into along z"""
    if nz is None:
        return ((nx + 63) // 64) * ((ny + 3) // 4)
    return lib().tacker_stencil_blocks(nx, ny, nz)


def ori_stencil(c0, c1, A0, Anext, stream=None):
    nz, ny, nx = A0.shape
    check(lib().tacker_ori_stencil(c0, c1, _ptr(A0), _ptr(Anext), nx, ny, nz, _stream(stream)),
          "tacker_ori_stencil")


def gptb_stencil(c0, c1, A0, Anext, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    nz, ny, nx = A0.shape
    if end is None:
        end = stencil_blocks(nx, ny, nz)
    check(lib().tacker_gptb_stencil(c0, c1, _ptr(A0), _ptr(Anext), nx, ny, nz, start, end, launch_grid,
                                    launch_block, _stream(stream)), "tacker_gptb_stencil")


def ori_lbm(src, dst, sx, sy, sz, stream=None):
    check(lib().tacker_ori_lbm(_ptr(src), _ptr(dst), sx, sy, sz, _stream(stream)), "tacker_ori_lbm")


def gptb_lbm(src, dst, sx, sy, sz, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    if end is None:
        end = sy * sz
    check(lib().tacker_gptb_lbm(_ptr(src), _ptr(dst), sx, sy, sz, start, end, launch_grid, launch_block,
                                _stream(stream)), "tacker_gptb_lbm")


def mriq_phimag(phiR, phiI, phiMag, stream=None):
    check(lib().tacker_mriq_phimag(_ptr(phiR), _ptr(phiI), _ptr(phiMag), phiR.numel(), _stream(stream)),
          "tacker_mriq_phimag")


def mriq_set_kvalues(kvals_np):
    """kvals_np: host numpy float32 [numK][4] = {Kx,Ky,Kz,PhiMag}."""
    import numpy as np
    kv = np.ascontiguousarray(kvals_np, np.float32)
    check(lib().tacker_mriq_set_kvalues(kv.ctypes.data, kv.shape[0]), "tacker_mriq_set_kvalues")


def mriq_blocks(numK, numX):
    """block positions of the GPTB form: voxel blocks x chunks of the k table"""
    return lib().tacker_mriq_blocks(numK, numX)


def ori_mriq(numK, x, y, z, Qr, Qi, stream=None):
    check(lib().tacker_ori_mriq(numK, _ptr(x), _ptr(y), _ptr(z), _ptr(Qr), _ptr(Qi), x.numel(),
                                _stream(stream)), "tacker_ori_mriq")


def gptb_mriq(numK, x, y, z, Qr, Qi, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    if end is None:
        end = mriq_blocks(numK, x.numel())
    check(lib().tacker_gptb_mriq(numK, _ptr(x), _ptr(y), _ptr(z), _ptr(Qr), _ptr(Qi), x.numel(), start,
                                 end, launch_grid, launch_block, _stream(stream)), "tacker_gptb_mriq")


def cp_initatoms(count=4000, volx=4096, voly=4096, volz=1, gridspacing=0.1):
    import numpy as np
    atoms = np.zeros((count, 4), np.float32)
    check(lib().tacker_cp_initatoms(atoms.ctypes.data, count, volx, voly, volz, gridspacing),
          "tacker_cp_initatoms")
    return atoms


def cp_set_atoms(atoms_np, zplane=0.0):
    import numpy as np
    a = np.ascontiguousarray(atoms_np, np.float32)
    check(lib().tacker_cp_set_atoms(a.ctypes.data, a.shape[0], zplane), "tacker_cp_set_atoms")


def cp_inv_sqrt_selftest(lo_bits=0x35800000, hi_bits=0x49800000):
    """floats in [lo_bits, hi_bits) for which the cp kernels' short 1/sqrt differs from 1.0f / sqrtf(x)"""
    n = C.c_ulonglong(0)
    check(lib().tacker_cp_inv_sqrt_selftest(lo_bits, hi_bits, C.byref(n)), "tacker_cp_inv_sqrt_selftest")
    return n.value


def cp_blocks(volx, voly):
    """block positions of the GPTB form: blocks of 128 x 8 points x parts of the unrolled x points"""
    return lib().tacker_cp_blocks(volx, voly)


def ori_cp(numatoms, gridspacing, grid, stream=None):
    voly, volx = grid.shape
    check(lib().tacker_ori_cp(numatoms, gridspacing, _ptr(grid), volx, voly, _stream(stream)),
          "tacker_ori_cp")


def gptb_cp(numatoms, gridspacing, grid, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    voly, volx = grid.shape
    if end is None:
        end = cp_blocks(volx, voly)
    check(lib().tacker_gptb_cp(numatoms, gridspacing, _ptr(grid), volx, voly, start, end, launch_grid,
                               launch_block, _stream(stream)), "tacker_gptb_cp")


def _gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream):
    M, K = A.shape
    N = B.shape[0]
    if tile_end is None:
        tile_end = (M // 64) * (N // 64)
    return [_ptr(A), _ptr(B), _ptr(Cm), M, N, K, tile_start, tile_end, _v(variant), launch_grid,
            launch_block, _stream(stream)]


def mix_tzgemm_stencil(c0, c1, A0, Anext, A, B, Cm, be_start=0, be_end=None, tile_start=0,
                       tile_end=None, variant=None, launch_grid=0, launch_block=0, stream=None):
    nz, ny, nx = A0.shape
    if be_end is None:
        be_end = stencil_blocks(nx, ny, nz)
    check(lib().tacker_mix_tzgemm_stencil(
        c0, c1, _ptr(A0), _ptr(Anext), nx, ny, nz, be_start, be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_stencil")


def mix_tzgemm_lbm(src, dst, sx, sy, sz, A, B, Cm, be_start=0, be_end=None, tile_start=0,
                   tile_end=None, variant=None, launch_grid=0, launch_block=0, stream=None):
    if be_end is None:
        be_end = sy * sz
    check(lib().tacker_mix_tzgemm_lbm(
        _ptr(src), _ptr(dst), sx, sy, sz, be_start, be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_lbm")
def mrif_rhophi(phiR, phiI, dR, dI, realRhoPhi, imagRhoPhi, stream=None):
    check(lib().tacker_mrif_rhophi(phiR.numel(), _ptr(phiR), _ptr(phiI), _ptr(dR), _ptr(dI), _ptr(realRhoPhi),
                                   _ptr(imagRhoPhi), _stream(stream)), "tacker_mrif_rhophi")


def mrif_set_kvalues(kvals_np):
    """kvals_np: host numpy float32 [numK][5] = {Kx,Ky,Kz,RhoPhiR,RhoPhiI}."""
    import numpy as np
    kv = np.ascontiguousarray(kvals_np, np.float32)
    check(lib().tacker_mrif_set_kvalues(kv.ctypes.data, kv.shape[0]), "tacker_mrif_set_kvalues")


def mrif_blocks(numK, numX):
    """block positions of the GPTB form: voxel blocks x chunks of the k table"""
    return lib().tacker_mrif_blocks(numK, numX)


def ori_mrif(numK, x, y, z, outR, outI, stream=None):
    check(lib().tacker_ori_mrif(numK, _ptr(x), _ptr(y), _ptr(z), _ptr(outR), _ptr(outI), x.numel(),
                                _stream(stream)), "tacker_ori_mrif")


def gptb_mrif(numK, x, y, z, outR, outI, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    if end is None:
        end = mrif_blocks(numK, x.numel())
    check(lib().tacker_gptb_mrif(numK, _ptr(x), _ptr(y), _ptr(z), _ptr(outR), _ptr(outI), x.numel(), start,
                                 end, launch_grid, launch_block, _stream(stream)), "tacker_gptb_mrif")


def mix_tzgemm_mrif(numK, x, y, z, outR, outI, A, B, Cm, be_start=0, be_end=None, tile_start=0,
                    tile_end=None, variant=None, launch_grid=0, launch_block=0, stream=None):
    if be_end is None:
        be_end = mrif_blocks(numK, x.numel())
    check(lib().tacker_mix_tzgemm_mrif(
        numK, _ptr(x), _ptr(y), _ptr(z), _ptr(outR), _ptr(outI), x.numel(), be_start, be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_mrif")


def _sgemm_dims(sA, sB, sC):
    """A is [K][M], B [K][N], C [N][M] (the reference's lda = M, ldb = N, ldc = M)"""
    K, M = sA.shape
    N = sB.shape[1]
    assert sB.shape[0] == K and tuple(sC.shape) == (N, M)
    return M, N, K


def sgemm_blocks(M, N, K):
    """block positions of the GPTB form: blocks of 128 x 16 of C x parts of the k loop"""
    return lib().tacker_sgemm_blocks(M, N, K)


def ori_sgemm(sA, sB, sC, stream=None):
    M, N, K = _sgemm_dims(sA, sB, sC)
    check(lib().tacker_ori_sgemm(_ptr(sA), _ptr(sB), _ptr(sC), M, N, K, _stream(stream)), "tacker_ori_sgemm")


def gptb_sgemm(sA, sB, sC, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    M, N, K = _sgemm_dims(sA, sB, sC)
    if end is None:
        end = sgemm_blocks(M, N, K)
    check(lib().tacker_gptb_sgemm(_ptr(sA), _ptr(sB), _ptr(sC), M, N, K, start, end, launch_grid, launch_block,
                                  _stream(stream)), "tacker_gptb_sgemm")


def mix_tzgemm_sgemm(sA, sB, sC, A, B, Cm, be_start=0, be_end=None, tile_start=0, tile_end=None, variant=None,
                     launch_grid=0, launch_block=0, stream=None):
    M, N, K = _sgemm_dims(sA, sB, sC)
    if be_end is None:
        be_end = sgemm_blocks(M, N, K)
    check(lib().tacker_mix_tzgemm_sgemm(
        _ptr(sA), _ptr(sB), _ptr(sC), M, N, K, be_start, be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_sgemm")


class CutcpInput:
    """prepare_input of the reference on host arrays, then on the device: the binned atoms (``bins``, with the
    padding bins), the address of bin (0, 0, 0), the neighbour list loaded into the device table, and an
    energy tensor [regions z][y][x][8][8][8] (``energies``)."""

    def __init__(self, atoms, lo, nx, ny, nz, h, cutoff, regions=None):
        import numpy as np
        import torch
        atoms = np.ascontiguousarray(atoms, np.float32).reshape(-1, 4)
        lo = np.ascontiguousarray(lo, np.float32)
        dims, pad, nlen, counts = (C.c_int * 3)(), C.c_int(), C.c_int(), (C.c_int * 2)()
        args = (atoms.ctypes.data, len(atoms), lo.ctypes.data, nx, ny, nz, h, cutoff)
        check(lib().tacker_cutcp_prepare_input(*args, dims, C.byref(pad), None, None, C.byref(nlen), counts),
              "tacker_cutcp_prepare_input")
        self.binDim = tuple(dims)
        self.padding = pad.value
        bins = np.zeros((dims[2], dims[1], dims[0], 8, 4), np.float32)
        nbr = np.zeros((nlen.value, 3), np.int32)
        check(lib().tacker_cutcp_prepare_input(*args, dims, C.byref(pad), bins.ctypes.data, nbr.ctypes.data,
                                               C.byref(nlen), counts), "tacker_cutcp_prepare_input")
        self.extra, self.excluded = counts[0], counts[1]
        self.nbr = nbr
        self.host_bins = bins
        self.h = float(h)
        self.bins = torch.from_numpy(bins).cuda()
        c = self.padding
        self.bin_zero = self.bins.data_ptr() + (((c * dims[1] + c) * dims[0] + c) * 32) * 4
        self.regions = regions or (-(-nx // 8), -(-ny // 8), -(-nz // 8))
        rx, ry, rz = self.regions
        self.energies = torch.zeros((rz, ry, rx, 8, 8, 8), device="cuda:0")
        self.load_neighbours()

    def load_neighbours(self):
        check(lib().tacker_cutcp_set_neighbours(self.nbr.ctypes.data, len(self.nbr)), "tacker_cutcp_set_neighbours")

    def blocks(self):
        """block positions of the GPTB form: regions x parts of the neighbour list (as loaded last)"""
        return lib().tacker_cutcp_blocks(*self.regions)

    def args(self, cutoff2, inv_cutoff2, energies=None):
        e = self.energies if energies is None else energies
        return (self.binDim[0], self.binDim[1], self.bin_zero, self.h, cutoff2, inv_cutoff2, _ptr(e)) + tuple(self.regions)


def ori_cutcp(inp, cutoff2, inv_cutoff2, energies=None, stream=None):
    check(lib().tacker_ori_cutcp(*inp.args(cutoff2, inv_cutoff2, energies), _stream(stream)), "tacker_ori_cutcp")


def gptb_cutcp(inp, cutoff2, inv_cutoff2, energies=None, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    check(lib().tacker_gptb_cutcp(*inp.args(cutoff2, inv_cutoff2, energies), start, inp.blocks() if end is None else end,
                                  launch_grid, launch_block, _stream(stream)), "tacker_gptb_cutcp")


def mix_tzgemm_cutcp(inp, cutoff2, inv_cutoff2, A, B, Cm, energies=None, be_start=0, be_end=None, tile_start=0,
                     tile_end=None, variant=None, launch_grid=0, launch_block=0, stream=None):
    check(lib().tacker_mix_tzgemm_cutcp(
        *inp.args(cutoff2, inv_cutoff2, energies), be_start, inp.blocks() if be_end is None else be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_cutcp")


def ori_cutcp_create(inp, cutoff2, inv_cutoff2, energies=None):
    return KernelHandle(lib().tacker_ori_cutcp_create(*inp.args(cutoff2, inv_cutoff2, energies)), "OriCUTCPKernel",
                        keep=(inp, energies))


def _fft_batches(data):
    """data: [batches][256][2] float32 device tensor (re, im), transformed in place"""
    if data.dim() != 3 or tuple(data.shape[1:]) != (256, 2) or not data.is_contiguous():
        raise ValueError("fft: data must be a contiguous [batches][256][2] float32 tensor")
    return data.shape[0]


def ori_fft(data, stream=None):
    check(lib().tacker_ori_fft(_ptr(data), _fft_batches(data), _stream(stream)), "tacker_ori_fft")


def gptb_fft(data, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    batches = _fft_batches(data)
    check(lib().tacker_gptb_fft(_ptr(data), batches, start, batches if end is None else end, launch_grid,
                                launch_block, _stream(stream)), "tacker_gptb_fft")


def mix_tzgemm_fft(data, A, B, Cm, be_start=0, be_end=None, tile_start=0, tile_end=None, variant=None,
                   launch_grid=0, launch_block=0, stream=None):
    batches = _fft_batches(data)
    check(lib().tacker_mix_tzgemm_fft(
        _ptr(data), batches, be_start, batches if be_end is None else be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_fft")


# ---- Rodinia partners: nn, hot3d, path
def nn_blocks(num_records):
    return lib().tacker_nn_blocks(num_records)


def _nn_records(locations, distances):
    """locations: [n][2] float32 {lat, lng}; distances: [n] float32"""
    if locations.dim() != 2 or locations.shape[1] != 2 or distances.numel() != locations.shape[0]:
        raise ValueError("nn: locations must be [n][2] and distances [n]")
    return locations.shape[0]


def ori_nn(locations, distances, lat, lng, stream=None):
    n = _nn_records(locations, distances)
    check(lib().tacker_ori_nn(_ptr(locations), _ptr(distances), n, lat, lng, _stream(stream)), "tacker_ori_nn")


def gptb_nn(locations, distances, lat, lng, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    n = _nn_records(locations, distances)
    check(lib().tacker_gptb_nn(_ptr(locations), _ptr(distances), n, lat, lng, start,
                               nn_blocks(n) if end is None else end, launch_grid, launch_block, _stream(stream)),
          "tacker_gptb_nn")


def mix_tzgemm_nn(locations, distances, lat, lng, A, B, Cm, be_start=0, be_end=None, tile_start=0, tile_end=None,
                  variant=None, launch_grid=0, launch_block=0, stream=None):
    n = _nn_records(locations, distances)
    check(lib().tacker_mix_tzgemm_nn(
        _ptr(locations), _ptr(distances), n, lat, lng, be_start, nn_blocks(n) if be_end is None else be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_nn")


def ori_nn_create(locations, distances, lat, lng):
    n = _nn_records(locations, distances)
    return KernelHandle(lib().tacker_ori_nn_create(_ptr(locations), _ptr(distances), n, lat, lng), "OriNNKernel",
                        keep=(locations, distances))


def hot3d_coefficients(nx, ny, nz):
    """{sdc, ce, cw, cn, cs, ct, cb, cc} of a step on nx x ny x nz cells, as float32 values."""
    out = (C.c_float * 8)()
    check(lib().tacker_hot3d_coefficients(nx, ny, nz, out), "tacker_hot3d_coefficients")
    return dict(zip(("sdc", "ce", "cw", "cn", "cs", "ct", "cb", "cc"), [float(v) for v in out]))


def hot3d_blocks(nx, ny):
    return (nx // 64) * (ny // 4)


def _hot3d_dims(p, t_in, t_out):
    """p, t_in, t_out: [nz][ny][nx] float32"""
    if t_in.dim() != 3 or tuple(p.shape) != tuple(t_in.shape) or tuple(t_out.shape) != tuple(t_in.shape):
        raise ValueError("hot3d: p, t_in and t_out must be [nz][ny][nx] tensors of one shape")
    nz, ny, nx = t_in.shape
    return nx, ny, nz


def ori_hot3d(p, t_in, t_out, stream=None):
    check(lib().tacker_ori_hot3d(_ptr(p), _ptr(t_in), _ptr(t_out), *_hot3d_dims(p, t_in, t_out), _stream(stream)),
          "tacker_ori_hot3d")


def gptb_hot3d(p, t_in, t_out, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    nx, ny, nz = _hot3d_dims(p, t_in, t_out)
    check(lib().tacker_gptb_hot3d(_ptr(p), _ptr(t_in), _ptr(t_out), nx, ny, nz, start,
                                  hot3d_blocks(nx, ny) if end is None else end, launch_grid, launch_block,
                                  _stream(stream)), "tacker_gptb_hot3d")


def mix_tzgemm_hot3d(p, t_in, t_out, A, B, Cm, be_start=0, be_end=None, tile_start=0, tile_end=None, variant=None,
                     launch_grid=0, launch_block=0, stream=None):
    nx, ny, nz = _hot3d_dims(p, t_in, t_out)
    check(lib().tacker_mix_tzgemm_hot3d(
        _ptr(p), _ptr(t_in), _ptr(t_out), nx, ny, nz, be_start, hot3d_blocks(nx, ny) if be_end is None else be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_hot3d")


def ori_hot3d_create(p, t_in, t_out):
    return KernelHandle(lib().tacker_ori_hot3d_create(_ptr(p), _ptr(t_in), _ptr(t_out), *_hot3d_dims(p, t_in, t_out)),
                        "OriHOT3DKernel", keep=(p, t_in, t_out))


def lava_blocks(boxes1d):
    return lib().tacker_lava_blocks(boxes1d)


def _lava_boxes1d(rv, qv, fv):
    """rv, fv: [n][4] float32 {v, x, y, z}; qv: [n] float32; n = 100 boxes1d^3"""
    n = qv.numel()
    boxes1d = round((n / 100) ** (1 / 3))
    if rv.dim() != 2 or rv.shape[1] != 4 or tuple(fv.shape) != tuple(rv.shape) or rv.shape[0] != n or \
            100 * boxes1d ** 3 != n:
        raise ValueError("lava: rv and fv must be [n][4], qv [n], n = 100 boxes1d^3")
    return boxes1d


def ori_lava(alpha, rv, qv, fv, stream=None):
    check(lib().tacker_ori_lava(alpha, _lava_boxes1d(rv, qv, fv), _ptr(rv), _ptr(qv), _ptr(fv), _stream(stream)),
          "tacker_ori_lava")


def gptb_lava(alpha, rv, qv, fv, start=0, end=None, launch_grid=0, launch_block=0, stream=None):
    b = _lava_boxes1d(rv, qv, fv)
    check(lib().tacker_gptb_lava(alpha, b, _ptr(rv), _ptr(qv), _ptr(fv), start, lava_blocks(b) if end is None else end,
                                 launch_grid, launch_block, _stream(stream)), "tacker_gptb_lava")


def mix_tzgemm_lava(alpha, rv, qv, fv, A, B, Cm, be_start=0, be_end=None, tile_start=0, tile_end=None, variant=None,
                    launch_grid=0, launch_block=0, stream=None):
    b = _lava_boxes1d(rv, qv, fv)
    check(lib().tacker_mix_tzgemm_lava(
        alpha, b, _ptr(rv), _ptr(qv), _ptr(fv), be_start, lava_blocks(b) if be_end is None else be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_lava")


def ori_lava_create(alpha, rv, qv, fv):
    return KernelHandle(lib().tacker_ori_lava_create(alpha, _lava_boxes1d(rv, qv, fv), _ptr(rv), _ptr(qv), _ptr(fv)),
                        "OriLAVAKernel", keep=(rv, qv, fv))


def path_blocks(cols, iteration):
    return lib().tacker_path_blocks(cols, iteration)


def _path_dims(wall, src, results):
    """wall: [rows - 1][cols] int32 (the grid without its first row); src, results: [cols] int32"""
    if wall.dim() != 2 or src.numel() != wall.shape[1] or results.numel() != wall.shape[1]:
        raise ValueError("path: wall must be [rows - 1][cols], src and results [cols]")
    return wall.shape[1], wall.shape[0] + 1


def ori_path(iteration, wall, src, results, start_step=0, stream=None):
    cols, rows = _path_dims(wall, src, results)
    check(lib().tacker_ori_path(iteration, _ptr(wall), _ptr(src), _ptr(results), cols, rows, start_step,
                                _stream(stream)), "tacker_ori_path")


def gptb_path(iteration, wall, src, results, start_step=0, start=0, end=None, launch_grid=0, launch_block=0,
              stream=None):
    cols, rows = _path_dims(wall, src, results)
    check(lib().tacker_gptb_path(iteration, _ptr(wall), _ptr(src), _ptr(results), cols, rows, start_step, start,
                                 path_blocks(cols, iteration) if end is None else end, launch_grid, launch_block,
                                 _stream(stream)), "tacker_gptb_path")


def mix_tzgemm_path(iteration, wall, src, results, A, B, Cm, start_step=0, be_start=0, be_end=None, tile_start=0,
                    tile_end=None, variant=None, launch_grid=0, launch_block=0, stream=None):
    cols, rows = _path_dims(wall, src, results)
    check(lib().tacker_mix_tzgemm_path(
        iteration, _ptr(wall), _ptr(src), _ptr(results), cols, rows, start_step, be_start,
        path_blocks(cols, iteration) if be_end is None else be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_path")


def ori_path_create(iteration, wall, src, results, start_step=0):
    cols, rows = _path_dims(wall, src, results)
    return KernelHandle(lib().tacker_ori_path_create(iteration, _ptr(wall), _ptr(src), _ptr(results), cols, rows,
                                                     start_step), "OriPATHKernel", keep=(wall, src, results))


def mix_tzgemm_mriq(numK, x, y, z, Qr, Qi, A, B, Cm, be_start=0, be_end=None, tile_start=0,
                    tile_end=None, variant=None, launch_grid=0, launch_block=0, stream=None):
    if be_end is None:
        be_end = mriq_blocks(numK, x.numel())
    check(lib().tacker_mix_tzgemm_mriq(
        numK, _ptr(x), _ptr(y), _ptr(z), _ptr(Qr), _ptr(Qi), x.numel(), be_start, be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_mriq")


def mix_tzgemm_cp(numatoms, gridspacing, grid, A, B, Cm, be_start=0, be_end=None, tile_start=0,
                  tile_end=None, variant=None, launch_grid=0, launch_block=0, stream=None):
    voly, volx = grid.shape
    if be_end is None:
        be_end = cp_blocks(volx, voly)
    check(lib().tacker_mix_tzgemm_cp(
        numatoms, gridspacing, _ptr(grid), volx, voly, be_start, be_end,
        *_gemm_args(A, B, Cm, tile_start, tile_end, variant, launch_grid, launch_block, stream)),
        "tacker_mix_tzgemm_cp")


def im2col(data_im, kernel, pad, stride, dilation, data_col, stream=None):
    Cc, H, W = data_im.shape
    check(lib().tacker_im2col(_ptr(data_im), Cc, H, W, kernel[0], kernel[1], pad[0], pad[1], stride[0],
                              stride[1], dilation[0], dilation[1], _ptr(data_col), _stream(stream)),
          "tacker_im2col")


def convert_fp32_to_fp16(out, inp, stream=None):
    check(lib().tacker_convert_fp32_to_fp16(_ptr(out), _ptr(inp), inp.numel(), _stream(stream)),
          "tacker_convert_fp32_to_fp16")


def mnk_from_conv_args(args14):
    a = (C.c_int * 14)(*args14)
    out = (C.c_int * 3)()
    lib().tacker_mnk_from_conv_args(a, out)
    return list(out)


def allocation_calls(library=None):
    """(tkMalloc calls, tkFree calls) of the library since it was loaded"""
    m, f = C.c_longlong(), C.c_longlong()
    check((library or lib()).tkAllocationCalls(C.byref(m), C.byref(f)), "tkAllocationCalls")
    return m.value, f.value


def spin_fail_flag():
    v = C.c_int()
    check(lib().tacker_spin_fail_flag(C.byref(v)), "tacker_spin_fail_flag")
    return v.value


# ----------------------------------------------------------------------------- object API
class KernelHandle:
    """Owner of one C++ Kernel object (Ori*, GPTBKernel or MixKernel)."""

    def __init__(self, handle, what, owned=True, keep=()):
        if not handle:
            raise TackerError(f"{what} failed: {lib().tacker_last_error().decode()}")
        self.handle = handle
        self.owned = owned
        self.keep = keep          # objects (tensors, handles) that must outlive this one

    def execute(self, stream=None):
        check(lib().tacker_kernel_execute(self.handle, _stream(stream)), "tacker_kernel_execute")

    def swap_buffers(self):
        check(lib().tacker_kernel_swap_buffers(self.handle), "tacker_kernel_swap_buffers")

    def info(self):
        out = (C.c_int * 8)()
        check(lib().tacker_kernel_info(self.handle, out), "tacker_kernel_info")
        keys = ("grid", "block", "ptb_start", "ptb_end", "nparams", "smem", "ori_grid_x", "ori_grid_y")
        return dict(zip(keys, out))

    def param(self, index, kind="ptr"):
        """Kernel parameter ``index`` as the launch passes it: a device address (``ptr``), ``int`` or ``float``."""
        ctype = {"ptr": C.c_void_p, "int": C.c_int, "float": C.c_float}[kind]
        out = ctype()
        check(lib().tacker_kernel_param(self.handle, index, C.byref(out), C.sizeof(ctype)), "tacker_kernel_param")
        return out.value or 0

    def use_module(self, module, function):
        """lmode DRIVER_LAUNCH: launch ``function`` of the registered code object ``module`` from now on."""
        check(lib().tacker_kernel_use_module(self.handle, module.encode(), function.encode()), "tacker_kernel_use_module")

    def set_range(self, *r):
        if len(r) == 2:
            check(lib().tacker_gptb_set_range(self.handle, *r), "tacker_gptb_set_range")
        else:
            check(lib().tacker_mix_set_range(self.handle, *r), "tacker_mix_set_range")

    def close(self):
        if self.owned and self.handle:
            lib().tacker_kernel_destroy(self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def register_module(name, path):
    """ModuleCenter::registerModule of the reference (src/ModuleCenter.cu:8-19) for a gfx950 code object."""
    check(lib().tacker_register_module(name.encode(), str(path).encode()), "tacker_register_module")


def module_has_function(module, function):
    return bool(lib().tacker_module_has_function(module.encode(), function.encode()))


def create_kernel(name):
    return KernelHandle(lib().tacker_create_kernel(name.encode()), f"createKernel({name})", owned=False)


def ori_stencil_create(c0, c1, A0, Anext):
    nz, ny, nx = A0.shape
    return KernelHandle(lib().tacker_ori_stencil_create(c0, c1, _ptr(A0), _ptr(Anext), nx, ny, nz),
                        "OriSTENCILKernel", keep=(A0, Anext))


def ori_lbm_create(src, dst, sx, sy, sz):
    return KernelHandle(lib().tacker_ori_lbm_create(_ptr(src), _ptr(dst), sx, sy, sz), "OriLBMKernel",
                        keep=(src, dst))


def ori_mriq_create(numK, x, y, z, Qr, Qi):
    return KernelHandle(lib().tacker_ori_mriq_create(numK, _ptr(x), _ptr(y), _ptr(z), _ptr(Qr), _ptr(Qi),
                                                     x.numel()), "OriMRIQKernel", keep=(x, y, z, Qr, Qi))


def ori_mrif_create(numK, x, y, z, outR, outI):
    return KernelHandle(lib().tacker_ori_mrif_create(numK, _ptr(x), _ptr(y), _ptr(z), _ptr(outR), _ptr(outI),
                                                     x.numel()), "OriMRIFKernel", keep=(x, y, z, outR, outI))


def ori_sgemm_create(sA, sB, sC):
    M, N, K = _sgemm_dims(sA, sB, sC)
    return KernelHandle(lib().tacker_ori_sgemm_create(_ptr(sA), _ptr(sB), _ptr(sC), M, N, K), "OriSGEMMKernel",
                        keep=(sA, sB, sC))


def ori_fft_create(data):
    return KernelHandle(lib().tacker_ori_fft_create(_ptr(data), _fft_batches(data)), "OriFFTKernel", keep=(data,))


def ori_cp_create(numatoms, gridspacing, grid):
    voly, volx = grid.shape
    return KernelHandle(lib().tacker_ori_cp_create(numatoms, gridspacing, _ptr(grid), volx, voly),
                        "OriCPKernel", keep=(grid,))


def ori_tzgemm_create(A, B, Cm, m=None, n=None, k=None):
    if A is not None:
        m, k = A.shape
        n = B.shape[0]
    return KernelHandle(lib().tacker_ori_tzgemm_create(_ptr(A), _ptr(B), _ptr(Cm), m, n, k),
                        "OriTZGEMMKernel", keep=(A, B, Cm))


def global_gemm_buffers():
    """(A, B, C device addresses, (bytes of A, B, C)) of the global operand buffers."""
    a, b, c = C.c_void_p(), C.c_void_p(), C.c_void_p()
    sizes = (C.c_longlong * 3)()
    check(lib().tacker_global_gemm_buffers(C.byref(a), C.byref(b), C.byref(c), sizes), "global_gemm_buffers")
    return a.value, b.value, c.value, tuple(sizes)


def gptb_create(ori, launch_grid=0, launch_block=0, start=0, end=0):
    return KernelHandle(lib().tacker_gptb_create(ori.handle, launch_grid, launch_block, start, end),
                        "GPTBKernel", keep=(ori,))


def mix_create(be_gptb, tz_gptb, be_start, be_end, tile_start, tile_end, variant=None, launch_grid=0,
               launch_block=0):
    return KernelHandle(lib().tacker_mix_create(be_gptb.handle, tz_gptb.handle, be_start, be_end,
                                                tile_start, tile_end, _v(variant), launch_grid,
                                                launch_block), "MixKernel", keep=(be_gptb, tz_gptb))


def be_pair_create(first_gptb, second_gptb, start1, end1, start2, end2, variant=None, launch_grid=0):
    """Fused launch of two best-effort GPTB kernels (first < second alphabetically)."""
    return KernelHandle(lib().tacker_be_pair_create(first_gptb.handle, second_gptb.handle, start1, end1,
                                                    start2, end2, _v(variant), launch_grid),
                        "MixKernel", keep=(first_gptb, second_gptb))


def mix_cublas_sgemm(mnk, be_gptb, start, end, stream=None, library=None):
    """mixcublasSgemm of the reference (src/TaskManager.cu:309-400): GEMM {M, N, K} on the global operand
    buffers fused with block positions [start, end) of a best-effort GPTB kernel."""
    l = library or lib()
    check(l.tacker_mix_cublas_sgemm((C.c_int * 3)(*mnk), be_gptb.handle, start, end,
                                    None if library else _stream(stream)), "mixcublasSgemm")


def mix_cudnn_convolution_forward(args14, be_gptb, start, end, stream=None, library=None):
    """mixcudnnConvolutionForward of the reference (src/TaskManager.cu:125-306)."""
    l = library or lib()
    check(l.tacker_mix_cudnn_convolution_forward((C.c_int * 14)(*args14), be_gptb.handle, start, end,
                                                 None if library else _stream(stream)), "mixcudnnConvolutionForward")


def create_mix_kernel(name):
    return KernelHandle(lib().tacker_create_mix_kernel(name.encode()), f"createMixKernel({name})", owned=False)


# ----------------------------------------------------------------------------- events
class Event:
    """tkEvent (hipEvent) recorded on the stream the kernels are launched on."""

    def __init__(self):
        self.h = C.c_void_p()
        lib().tkEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        lib().tkEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        lib().tkEventSynchronize.argtypes = [C.c_void_p]
        lib().tkEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        lib().tkEventDestroy.argtypes = [C.c_void_p]
        check(lib().tkEventCreate(C.byref(self.h)), "tkEventCreate")

    def record(self, stream=None):
        check(lib().tkEventRecord(self.h, _stream(stream)), "tkEventRecord")

    def synchronize(self):
        check(lib().tkEventSynchronize(self.h), "tkEventSynchronize")

    def elapsed_ms(self, later):
        ms = C.c_float()
        check(lib().tkEventElapsedTime(C.byref(ms), self.h, later.h), "tkEventElapsedTime")
        return ms.value

    def __del__(self):
        try:
            if self.h:
                lib().tkEventDestroy(self.h)
        except Exception:
            pass


def device_to_host(ptr, shape, dtype, library=None):
    """tkMemcpy device -> host of a raw device pointer into a fresh numpy array."""
    import numpy as np
    out = np.empty(shape, dtype)
    l = library or lib()
    rc = l.tkMemcpy(out.ctypes.data, ptr, out.nbytes, 2)
    if rc:
        raise TackerError(f"tkMemcpy failed ({rc})")
    return out


# ----------------------------------------------------------------------------- LC task + scheduler
REPORT_KEYS = ("lc_solo_ms", "be1_solo_ms", "be2_solo_ms", "be_blocks_executed", "mix_times",
               "mixable_times", "time_earned_ms", "qos_headroom_left_ms", "stage1_be_ms", "stage2_be_ms",
               "be_task_finish_num", "n_colocated", "n_solo")


class QueryGraph:
    """A recorded query (tkGraphExec_t): ``launch(raw_stream)`` enqueues all its kernels at once."""

    def __init__(self, library, handle):
        self.l, self.h = library, handle

    def launch(self, raw_stream):
        rc = self.l.tkGraphLaunch(self.h, raw_stream)
        if rc:
            raise TackerError(f"tkGraphLaunch failed ({rc})")

    def close(self):
        if self.h:
            self.l.tkGraphExecDestroy(self.h)
            self.h = None


class LcTask:
    """createTask(model): the latency-critical job (VGG16 at batch 1)."""

    def __init__(self, model="vgg16", height=0, width=0, library=None):
        self.l = library or lib()
        self.h = self.l.tacker_task_create(model.encode(), height, width)
        if not self.h:
            raise TackerError(f"createTask({model}) failed: {self.l.tacker_last_error().decode()}")

    def execute(self, stream=None, raw_stream=...):
        st = raw_stream if raw_stream is not ... else _stream(stream)
        rc = self.l.tacker_task_execute(self.h, st)
        if rc:
            raise TackerError(f"task execute failed ({rc}): {self.l.tacker_last_error().decode()}")

    def stage_input(self):
        """Task::initExecution alone: the query's input copied to the device (synchronous)."""
        rc = self.l.tacker_task_stage_input(self.h)
        if rc:
            raise TackerError(f"task stage_input failed ({rc}): {self.l.tacker_last_error().decode()}")

    def capture(self, raw_stream):
        """The task's launches recorded from ``raw_stream`` (a tkStream_t, not the null stream) into
        a ``QueryGraph``; run ``execute`` once before so that every buffer exists."""
        exec_ = C.c_void_p()
        rc = self.l.tacker_task_capture(self.h, raw_stream, C.byref(exec_))
        if rc:
            raise TackerError(f"task capture failed ({rc}): {self.l.tacker_last_error().decode()}")
        return QueryGraph(self.l, exec_)

    def kernels(self):
        out = []
        for idx in range(self.l.tacker_task_kernel_count(self.h)):
            name = C.create_string_buffer(128)
            mix, n = C.c_int(), C.c_int()
            args = (C.c_int * 14)()
            self.l.tacker_task_kernel_info(self.h, idx, name, 128, C.byref(mix), args, C.byref(n))
            out.append({"name": name.value.decode(), "mixable": mix.value, "args": list(args)[:n.value]})
        return out

    def activation(self, conv_index):
        p = C.c_void_p()
        dims = (C.c_int * 4)()
        rc = self.l.tacker_task_activation(self.h, conv_index, C.byref(p), dims)
        if rc:
            raise TackerError(self.l.tacker_last_error().decode())
        return p.value, tuple(dims)

    def conv_params(self, conv_index):
        """(weights f16 [Np][Kp], bias f32 [Np]) of a convolution (0..12) or a fully connected layer
        (13..15; the last has no bias: zeros), copied to the host."""
        import numpy as np
        w, b = C.c_void_p(), C.c_void_p()
        dims = (C.c_int * 2)()
        rc = self.l.tacker_task_conv_params(self.h, conv_index, C.byref(w), C.byref(b), dims)
        if rc:
            raise TackerError(self.l.tacker_last_error().decode())
        return (device_to_host(w.value, (dims[0], dims[1]), np.float16, self.l),
                device_to_host(b.value, (dims[0],), np.float32, self.l) if b.value else np.zeros(dims[0], np.float32))

    def logits(self):
        p = C.c_void_p()
        stride, n = C.c_long(), C.c_int()
        rc = self.l.tacker_task_logits(self.h, C.byref(p), C.byref(stride), C.byref(n))
        if rc:
            raise TackerError(self.l.tacker_last_error().decode())
        return p.value, stride.value, n.value

    def host_input(self):
        import numpy as np
        p = C.c_void_p()
        nbytes = C.c_int()
        self.l.tacker_task_input(self.h, C.byref(p), C.byref(nbytes))
        buf = (C.c_float * (nbytes.value // 4)).from_address(p.value)
        return np.frombuffer(buf, dtype=np.float32)

    def close(self):
        if self.h:
            self.l.tacker_task_destroy(self.h)
            self.h = None


class TaskManager:
    """TaskManager(lc_task, be1, be2) with the reference's constants exposed."""

    def __init__(self, task, be1, be2=None, library=None):
        self.l = library or lib()
        self.task = task
        self.h = self.l.tacker_task_manager_create(task.h, be1.encode(), be2.encode() if be2 else None)
        if not self.h:
            raise TackerError(f"TaskManager failed: {self.l.tacker_last_error().decode()}")

    def configure(self, qos_budget_ms=-1.0, guard_ms=-1.0, warmup=-1, profile=-1, queries=-1, verbose=-1):
        self.l.tacker_task_manager_configure(self.h, qos_budget_ms, guard_ms, warmup, profile, queries, verbose)

    def run(self, mode="aker", stream=None, second_stage=False, raw_stream=...):
        st = raw_stream if raw_stream is not ... else _stream(stream)
        rc = self.l.tacker_task_manager_run(self.h, 0 if mode == "aker" else 1, st, 1 if second_stage else 0)
        if rc:
            raise TackerError(f"TaskManager run failed ({rc}): {self.l.tacker_last_error().decode()}")
        return self.report()

    def report(self):
        out = (C.c_float * 13)()
        self.l.tacker_task_manager_report(self.h, out)
        return dict(zip(REPORT_KEYS, out))

    def set_fusion_strikes(self, limit):
        check(self.l.tacker_task_manager_set_fusion_strikes(self.h, limit), "set_fusion_strikes")

    def set_calibration(self, on=True, max_stretch=0.10):
        check(self.l.tacker_task_manager_set_calibration(self.h, 1 if on else 0, max_stretch), "set_calibration")

    def set_calibration_budget(self, query_stretch=0.15, passes=3):
        """calibration chooses per query: the fused launches may add ``query_stretch`` of the query's solo
        time in total (0 = the best count per kernel); ``passes`` timed launches per option"""
        check(self.l.tacker_task_manager_set_calibration_budget(self.h, query_stretch, passes), "set_calibration_budget")

    def set_calibration_variants(self, variants=("default", "wave_256")):
        """forms of the fused kernel the calibration pass tries per LC kernel ("default" = kinfo's)"""
        check(self.l.tacker_task_manager_set_calibration_variants(self.h, ",".join(variants).encode()),
              "set_calibration_variants")

    def calibrated_blocks(self):
        buf = (C.c_int * 4096)()
        n = self.l.tacker_task_manager_calibrated_blocks(self.h, buf, 4096)
        return list(buf[:max(n, 0)])

    def calibrated_variants(self):
        """the form kept per LC kernel by the last calibrated run ("" = the pair's default)"""
        out = []
        buf = C.create_string_buffer(64)
        for k in range(len(self.calibrated_blocks())):
            if self.l.tacker_task_manager_calibrated_variant(self.h, k, buf, 64) < 0:
                break
            out.append(buf.value.decode())
        return out

    def fusion_disabled(self):
        return self.l.tacker_task_manager_fusion_disabled(self.h)

    def be_mix_ms(self):
        return self.l.tacker_task_manager_be_mix_ms(self.h)

    def set_end_to_end(self, queries):
        check(self.l.tacker_task_manager_set_end_to_end(self.h, queries), "set_end_to_end")

    LATENCY_KINDS = {"colocated": 0, "solo": 1, "e2e_colocated": 2, "e2e_solo": 3,
                     "e2e_colocated_wall": 4, "e2e_solo_wall": 5, "e2e_graph": 6, "e2e_graph_wall": 7}

    def latencies(self, solo=False, kind=None):
        """Per-query latencies in ms.  ``kind`` picks one of LATENCY_KINDS: the sums of per-kernel
        intervals (``colocated``, ``solo``) or whole queries timed end to end by events / by the
        host clock (``e2e_*``, after ``set_end_to_end``).  Without it, ``solo`` picks between the
        first two."""
        which = self.LATENCY_KINDS[kind] if kind is not None else (1 if solo else 0)
        cap = 1 << 16
        buf = (C.c_float * cap)()
        n = self.l.tacker_task_manager_latencies(self.h, which, buf, cap)
        return list(buf[:max(n, 0)])

    def close(self):
        if self.h:
            self.l.tacker_task_manager_destroy(self.h)
            self.h = None
