"""gfx950 stand-in for the `ista_daslab_cuda_micro_adam` extension module of the package
ista-daslab-optimizers-cuda: same function names, argument order and in-place semantics as
the calls in ista_daslab_optimizers/micro_adam/micro_adam.py:190, :231, :267, :277-291, :298,
:313, :316, :322, on top of libmicroadam_hip.so.
"""
import torch

from ista_daslab_optimizers import _hip


def _stats_len(d, q):
    return (d + q - 1) // q


def _check_quant(d, q, xq, xmin, xmax, x):
    if xq.numel() < (d + 1) // 2 or x.numel() < d:
        raise RuntimeError("quantisation buffers shorter than d")
    if xmin.numel() < _stats_len(d, q) or xmax.numel() < _stats_len(d, q):
        raise RuntimeError("min/max statistics shorter than the number of quantisation blocks")


def asymm_block_quant(d, q_block_size, xq, xmin, xmax, x):
    _check_quant(d, q_block_size, xq, xmin, xmax, x)
    rc = _hip.lib.ma_asymm_block_quant(d, q_block_size, _hip.dev_ptr(xq, torch.uint8, "xq"),
                                       _hip.dev_ptr(xmin, torch.bfloat16, "xmin"),
                                       _hip.dev_ptr(xmax, torch.bfloat16, "xmax"),
                                       _hip.dev_ptr(x, None, "x"), _hip.dtype_tag(x),
                                       _hip.stream_ptr())
    _hip.check(rc, "asymm_block_quant")


def asymm_block_quant_inv(d, q_block_size, xq, xmin, xmax, x, alpha):
    _check_quant(d, q_block_size, xq, xmin, xmax, x)
    rc = _hip.lib.ma_asymm_block_quant_inv(d, q_block_size, _hip.dev_ptr(xq, torch.uint8, "xq"),
                                           _hip.dev_ptr(xmin, torch.bfloat16, "xmin"),
                                           _hip.dev_ptr(xmax, torch.bfloat16, "xmax"),
                                           _hip.dev_ptr(x, None, "x"), float(alpha),
                                           _hip.dtype_tag(x), _hip.stream_ptr())
    _hip.check(rc, "asymm_block_quant_inv")


def compute_microadam_update(blocks, threads, carveout, t, beta1, beta2, eps, d_block_size,
                             k_block_size, d, m, k, indices, values, out):
    if indices.numel() < m * k or values.numel() < m * k or out.numel() < d:
        raise RuntimeError("compute_microadam_update: window or output shorter than m*k / d")
    rc = _hip.lib.ma_compute_microadam_update(
        int(blocks), int(threads), int(carveout), int(t), float(beta1), float(beta2), float(eps),
        d_block_size, k_block_size, d, m, k, _hip.dev_ptr(indices, torch.int16, "indices"),
        _hip.dev_ptr(values, torch.bfloat16, "values"), _hip.dev_ptr(out, None, "out"),
        _hip.dtype_tag(out), _hip.stream_ptr())
    _hip.check(rc, "compute_microadam_update")
