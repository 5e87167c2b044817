"""ctypes binding of libmicroadam_hip.so (the C ABI declared in include/microadam_hip.h).

The library is built in-tree by csrc/Makefile (hipcc, gfx950) and loaded from this package's
directory.  There is no CPU fallback: if the library is missing, importing this module
raises, and a failed launch raises RuntimeError with the library's own message.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmicroadam_hip.so")

MA_F32, MA_BF16 = 0, 1
MA_ERR_ARG = -1
MA_ERR_NOT_FUSABLE = -5
MA_ERR_LDS = -6
MA_ERR_WORKSPACE = -7
MA_STATIC_WORKSPACE_BYTES = 16 << 20
MA_ROUTE_FUSED, MA_ROUTE_DENSIFIED, MA_ROUTE_SPANNING, MA_ROUTE_QUANT_ERR = 0, 1, 2, 3
MA_MAX_WINDOW = 64


class MaTensor(ctypes.Structure):
    """struct ma_tensor"""
    _fields_ = [("p", ctypes.c_void_p), ("g", ctypes.c_void_p), ("error", ctypes.c_void_p),
                ("min_vals", ctypes.c_void_p), ("max_vals", ctypes.c_void_p),
                ("I", ctypes.c_void_p), ("V", ctypes.c_void_p), ("d", ctypes.c_int64),
                ("k", ctypes.c_int64), ("lr", ctypes.c_double), ("weight_decay", ctypes.c_double),
                ("index", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("quant_err", ctypes.c_void_p), ("row_cuts", ctypes.c_void_p)]


class MaHyper(ctypes.Structure):
    """struct ma_hyper"""
    _fields_ = [("t", ctypes.c_int64), ("m", ctypes.c_int32), ("dtype", ctypes.c_int32),
                ("quant_block_size", ctypes.c_int64), ("d_block_size", ctypes.c_int64),
                ("k_init", ctypes.c_double), ("beta1", ctypes.c_double),
                ("beta2", ctypes.c_double), ("eps", ctypes.c_double)]


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C ista-daslab-optimizers_amd/csrc` "
            "(hipcc, gfx950). MicroAdam has no CPU or PyTorch fallback.")
    L = ctypes.CDLL(LIB_PATH)
    vp, i64, ci, f32, f64 = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float,
                             ctypes.c_double)
    sig = {
        "ma_error_string": (ctypes.c_char_p, [ci]),
        "ma_get_sm_count": (ci, []),
        "ma_get_max_floats_for_shared_memory_per_thread_block": (ci, []),
        "ma_copy_values": (ci, [i64, i64, i64, i64, vp, vp, vp, ci, ci, vp]),
        "ma_zerorize_block_components": (ci, [vp, vp, i64, i64, i64, i64, ci, vp]),
        "ma_asymm_block_quant": (ci, [i64, i64, vp, vp, vp, vp, ci, vp]),
        "ma_asymm_block_quant_inv": (ci, [i64, i64, vp, vp, vp, vp, f32, ci, vp]),
        "ma_compute_microadam_update": (ci, [ci, ci, ci, i64, f64, f64, f64, i64, i64, i64, i64,
                                             i64, vp, vp, vp, ci, vp]),
        "ma_block_topk": (ci, [i64, i64, i64, i64, vp, vp, vp, ci, ci, vp]),
        "ma_block_minmax": (ci, [i64, i64, vp, vp, vp, ci, vp]),
        "ma_param_update": (ci, [i64, vp, vp, f32, ci, f32, ci, vp]),
        "ma_fused_step": (ci, [ctypes.POINTER(MaTensor), ci, ctypes.POINTER(MaHyper), vp]),
        "ma_fused_step_check": (ci, [ctypes.POINTER(MaTensor), ctypes.POINTER(MaHyper)]),
        "ma_fused_step_row_cuts": (ctypes.c_int64, [ctypes.POINTER(MaTensor),
                                                    ctypes.POINTER(MaHyper)]),
        "ma_fused_step_densified": (ci, [ctypes.POINTER(MaTensor), ci, ctypes.POINTER(MaHyper),
                                         ctypes.c_double, vp]),
        "ma_fused_step_quant_err": (ci, [ctypes.POINTER(MaTensor), ci, ctypes.POINTER(MaHyper),
                                         vp]),
        "ma_logged_step": (ci, [ci, ctypes.POINTER(MaTensor), ci, ctypes.POINTER(MaHyper),
                                ctypes.c_double, vp, i64, vp, i64, vp, vp]),
        "ma_logged_step_partials": (i64, [ctypes.POINTER(MaTensor), ci, ctypes.POINTER(MaHyper)]),
        "ma_spanning_step": (ci, [ctypes.POINTER(MaTensor), ci, ctypes.POINTER(MaHyper),
                                   ctypes.c_double, vp, ctypes.c_int64, vp]),
        "ma_spanning_step_static": (ci, [ctypes.POINTER(MaTensor), ci, ctypes.POINTER(MaHyper),
                                          ctypes.c_double, vp]),
        "ma_spanning_step_workspace": (ctypes.c_int64, [ctypes.POINTER(MaTensor), ci,
                                                         ctypes.POINTER(MaHyper)]),
        "ma_spanning_step_check": (ci, [ctypes.POINTER(MaTensor), ctypes.POINTER(MaHyper),
                                         ctypes.c_double]),
        "ma_sparse_scalar_products": (ci, [i64, i64, i64, i64, i64, vp, ci, vp, vp, ci, vp, vp,
                                           i64, vp]),
        "ma_sparse_scalar_products_workspace": (ci, [i64, i64, i64, i64, i64,
                                                     ctypes.POINTER(ctypes.c_int64)]),
        "ma_sparse_linear_combination": (ci, [i64, i64, i64, i64, i64, vp, vp, vp, ci, vp, ci,
                                              vp]),
        "ma_copy_values_typed": (ci, [i64, i64, i64, i64, vp, vp, vp, ci, ci, ci, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    return L


lib = _load()
EXPORTS = ("ma_error_string", "ma_get_sm_count",
           "ma_get_max_floats_for_shared_memory_per_thread_block", "ma_copy_values",
           "ma_zerorize_block_components", "ma_asymm_block_quant", "ma_asymm_block_quant_inv",
           "ma_compute_microadam_update", "ma_block_topk", "ma_block_minmax", "ma_param_update",
           "ma_fused_step", "ma_fused_step_check", "ma_fused_step_row_cuts",
           "ma_fused_step_densified",
           "ma_fused_step_quant_err", "ma_logged_step", "ma_logged_step_partials",
           "ma_spanning_step", "ma_spanning_step_static", "ma_spanning_step_workspace",
           "ma_spanning_step_check", "ma_sparse_scalar_products",
           "ma_sparse_scalar_products_workspace", "ma_sparse_linear_combination",
           "ma_copy_values_typed")


def error_string(code):
    return lib.ma_error_string(int(code)).decode()


def check(code, what):
    """Negative codes reject the call before anything was launched.  A positive code is the
    hipError_t of a launch the runtime refused: launches before it have run, so a step call may
    be part-way applied and must not be repeated."""
    if code > 0:
        raise RuntimeError(f"{what}: the HIP runtime refused a launch: {error_string(code)} "
                           f"(hipError_t {code}); earlier launches of the call have run, so "
                           "restore the optimizer from a checkpoint instead of stepping again")
    if code != 0:
        raise RuntimeError(f"{what} failed: {error_string(code)} (code {code})")


def dtype_tag(t):
    import torch
    if t.dtype == torch.float32:
        return MA_F32
    if t.dtype == torch.bfloat16:
        return MA_BF16
    raise TypeError(f"MicroAdam kernels take float32 or bfloat16 tensors, got {t.dtype}")


def stream_ptr():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def dev_ptr(t, dtype=None, name="tensor"):
    """Device address of a contiguous CUDA/HIP tensor, with the checks the kernels rely on."""
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (got {t.device}); MicroAdam has no CPU path")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    return ctypes.c_void_p(t.data_ptr())
