"""gfx950 stand-in for the `ista_daslab_cuda_tools` extension module of the package
ista-daslab-optimizers-cuda: same function names, argument order and in-place semantics as
the calls in ista_daslab_optimizers/micro_adam/micro_adam.py:40, :43, :202-209, :214 and
sparse_mfac/sparse_core_mfac_w_ef.py:105-124, on top of libmicroadam_hip.so.  With this
directory on sys.path the reference's own micro_adam.py imports it unchanged.
"""
import torch

from ista_daslab_optimizers import _hip


def get_sm_count():
    n = _hip.lib.ma_get_sm_count()
    if n <= 0:
        raise RuntimeError("no HIP device")
    return n


def get_max_floats_for_shared_memory_per_thread_block():
    return _hip.lib.ma_get_max_floats_for_shared_memory_per_thread_block()


def copy_values(d, k, d_block_size, k_block_size, indices, inp, out, direction):
    dense = inp if direction == 1 else out
    sparse = out if direction == 1 else inp
    if indices.numel() < k or sparse.numel() < k or dense.numel() < d:
        raise RuntimeError("copy_values: tensor shorter than d / k")
    if sparse.dtype == torch.bfloat16:
        rc = _hip.lib.ma_copy_values(d, k, d_block_size, k_block_size,
                                     _hip.dev_ptr(indices, torch.int16, "indices"),
                                     _hip.dev_ptr(inp, None, "inp"),
                                     _hip.dev_ptr(out, None, "out"), int(direction),
                                     _hip.dtype_tag(dense), _hip.stream_ptr())
    else:  # Sparse M-FAC with use_bf16 = False keeps fp32 values
        rc = _hip.lib.ma_copy_values_typed(d, k, d_block_size, k_block_size,
                                           _hip.dev_ptr(indices, torch.int16, "indices"),
                                           _hip.dev_ptr(inp, None, "inp"),
                                           _hip.dev_ptr(out, None, "out"), int(direction),
                                           _hip.dtype_tag(dense), _hip.dtype_tag(sparse),
                                           _hip.stream_ptr())
    _hip.check(rc, "copy_values")


def zerorize_block_components(vector, indices, d, k, d_block_size, k_block_size):
    if indices.numel() < k or vector.numel() < d:
        raise RuntimeError("zerorize_block_components: tensor shorter than d / k")
    rc = _hip.lib.ma_zerorize_block_components(_hip.dev_ptr(vector, None, "vector"),
                                               _hip.dev_ptr(indices, torch.int16, "indices"), d, k,
                                               d_block_size, k_block_size,
                                               _hip.dtype_tag(vector), _hip.stream_ptr())
    _hip.check(rc, "zerorize_block_components")
