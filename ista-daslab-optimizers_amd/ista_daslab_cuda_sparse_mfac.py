"""gfx950 stand-in for the two functions of the `ista_daslab_cuda_sparse_mfac` extension module
(package ista-daslab-optimizers-cuda) that work on the window layout MicroAdam shares with
Sparse M-FAC: same names, argument order and in-place semantics as the calls in
ista_daslab_optimizers/sparse_mfac/sparse_core_mfac_w_ef.py:188-201 (SP) and :208-221 (LCG),
on top of libmicroadam_hip.so.
"""
import ctypes

import torch

from ista_daslab_optimizers import _hip

_workspace = {}  # device index -> uint8 tensor holding SP's per-block partial sums


def _window(d, m, k, I, V, use_bf16):
    want = torch.bfloat16 if use_bf16 else torch.float32
    if V.dtype != want:
        raise TypeError(f"use_bf16={use_bf16} but the values are {V.dtype}")
    if I.dim() != 2 or I.shape[1] != k or V.shape != I.shape or I.shape[0] < m:
        raise RuntimeError("I and V must be [rows >= m, k]")
    return _hip.dev_ptr(I, torch.int16, "I"), _hip.dev_ptr(V, want, "V")


def SP(blocks, threads, version, d, m, k, d_block_size, k_block_size, g, I, V, out, use_bf16):
    """out[i] += <row i of the window, g> for i < m (the launch shape and kernel version of the
    CUDA module are accepted and ignored)."""
    del blocks, threads, version
    pI, pV = _window(d, m, k, I, V, use_bf16)
    if g.numel() < d or out.numel() < m:
        raise RuntimeError("SP: g shorter than d or out shorter than m")
    need = ctypes.c_int64()
    _hip.check(_hip.lib.ma_sparse_scalar_products_workspace(d, m, k, d_block_size, k_block_size,
                                                            ctypes.byref(need)), "SP")
    ws = _workspace.get(g.device.index)
    if ws is None or ws.numel() < need.value:
        ws = _workspace[g.device.index] = torch.empty(max(need.value, 4), dtype=torch.uint8,
                                                      device=g.device)
    rc = _hip.lib.ma_sparse_scalar_products(
        d, m, k, d_block_size, k_block_size, _hip.dev_ptr(g, None, "g"), _hip.dtype_tag(g), pI, pV,
        _hip.dtype_tag(V), _hip.dev_ptr(out, torch.float32, "out"), _hip.dev_ptr(ws), ws.numel(),
        _hip.stream_ptr())
    _hip.check(rc, "SP")


def LCG(blocks, threads, version, d, m, k, d_block_size, k_block_size, M, I, V, out, use_bf16):
    """out += sum over i < m of M[i] * (row i of the window scattered to length d)."""
    del blocks, threads, version
    pI, pV = _window(d, m, k, I, V, use_bf16)
    if out.numel() < d or M.numel() < m:
        raise RuntimeError("LCG: out shorter than d or M shorter than m")
    rc = _hip.lib.ma_sparse_linear_combination(
        d, m, k, d_block_size, k_block_size, _hip.dev_ptr(M, torch.float32, "M"), pI, pV,
        _hip.dtype_tag(V), _hip.dev_ptr(out, None, "out"), _hip.dtype_tag(out), _hip.stream_ptr())
    _hip.check(rc, "LCG")
