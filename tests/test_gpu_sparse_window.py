"""GPU parity of Sparse M-FAC's kernels over the window layout (scalar products, linear
combination, copy_values with fp32 values) against the CPU oracle, through the C ABI's ctypes
binding and the `ista_daslab_cuda_sparse_mfac` / `ista_daslab_cuda_tools` stand-ins.

The linear combination is bit-exact (its order of additions is fixed).  The scalar products are
fp32 sums whose order is the device's own: they are compared with the oracle's double sums
within 2e-6 of the sum of the absolute terms (products rounded to fp32, butterfly sums of up to
a few thousand partial sums), and must be bit-identical from call to call.
"""
import math

import numpy as np
import pytest
import torch

from gpu_util import to_np, to_torch

pytestmark = pytest.mark.gpu

SP_TOL = 2e-6


@pytest.fixture(scope="module")
def mods():
    import ista_daslab_cuda_sparse_mfac
    import ista_daslab_cuda_tools
    return ista_daslab_cuda_tools, ista_daslab_cuda_sparse_mfac


def _geometry(d, dbs, k_init):
    full, tail0 = (1, d) if d < dbs else (d // dbs, (d // dbs) * dbs)
    kb = math.ceil(min(dbs, d) * k_init)
    lens = [min(dbs, d)] * full + ([d - tail0] if tail0 < d else [])
    kbs = [kb] * full + ([math.ceil((d - tail0) * k_init)] if tail0 < d else [])
    return lens, kbs, kb


def _window(seed, d, dbs, k_init, m, dtype):
    """m rows of distinct block-relative indices per top-k block, and values of `dtype`."""
    lens, kbs, kb = _geometry(d, dbs, k_init)
    gen = torch.Generator().manual_seed(seed)
    cols = []
    for ln, kk in zip(lens, kbs):
        cols.append(torch.rand(m, ln, generator=gen).argsort(dim=1)[:, :kk])
    I = torch.cat(cols, dim=1).to(torch.int16)
    V = torch.randn(I.shape, generator=gen).to(dtype)
    return I, V, I.shape[1], kb


# d, d_block_size, k_init, window rows, live rows
SHAPES = [
    (20480 * 3 + 4096, 20480, 0.01, 32, 20),   # MicroAdam's block size, a tail block
    (1000, 256, 0.05, 8, 8),
    (300, 512, 0.1, 4, 3),                     # one short block
    (20480 * 2, 20480, 0.5, 6, 6),             # rows longer than one batch of entries
    (4096 * 5 + 11, 4096, 0.02, 130, 129),     # more rows than waves, odd tail
    (32768 * 2, 32768, 0.01, 5, 5),            # the longest block the int16 indices allow
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("d,dbs,k_init,m,rows", SHAPES)
def test_scalar_products(mods, oracle, dtype, d, dbs, k_init, m, rows):
    _, smf = mods
    I, V, k, kb = _window(d, d, dbs, k_init, m, dtype)
    gen = torch.Generator().manual_seed(d + 1)
    g = torch.randn(d, generator=gen).to(dtype)
    want = np.zeros(m)
    oracle.sparse_scalar_products(d, rows, k, dbs, kb, to_np(g), to_np(I), to_np(V), want)
    pos = (torch.arange(k) // kb) * dbs + I.long()
    mass = (V.double().abs() * g.double()[pos].abs()).sum(dim=1).numpy()
    Id, Vd, gd = I.cuda(), V.cuda(), g.cuda()
    outs = []
    for _ in range(2):
        out = torch.zeros(m, dtype=torch.float32, device="cuda")
        smf.SP(256, 1024, 23, d, rows, k, dbs, kb, gd, Id, Vd, out, int(dtype == torch.bfloat16))
        outs.append(out.cpu().numpy())
    assert np.array_equal(outs[0], outs[1])
    assert np.all(np.abs(outs[0][:rows] - want[:rows]) <= SP_TOL * mass[:rows] + 1e-30)
    assert np.all(outs[0][rows:] == 0)


def test_scalar_products_accumulate_into_out(mods, oracle):
    _, smf = mods
    d, dbs, m = 5000, 1024, 4
    I, V, k, kb = _window(1, d, dbs, 0.02, m, torch.bfloat16)
    g = torch.randn(d, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    zero = torch.zeros(m, dtype=torch.float32, device="cuda")
    smf.SP(0, 0, 23, d, m, k, dbs, kb, g.cuda(), I.cuda(), V.cuda(), zero, 1)
    out = torch.full((m,), 3.0, dtype=torch.float32, device="cuda")
    smf.SP(0, 0, 23, d, m, k, dbs, kb, g.cuda(), I.cuda(), V.cuda(), out, 1)
    assert torch.equal(out, zero + 3.0)


@pytest.mark.parametrize("vdtype,odtype", [(torch.bfloat16, torch.bfloat16),
                                           (torch.float32, torch.float32),
                                           (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("d,dbs,k_init,m,rows", SHAPES)
def test_linear_combination(mods, oracle, hip_lib, vdtype, odtype, d, dbs, k_init, m, rows):
    _, smf = mods
    I, V, k, kb = _window(d + 7, d, dbs, k_init, m, vdtype)
    gen = torch.Generator().manual_seed(d + 2)
    coef = torch.randn(m, generator=gen)
    start = (torch.randn(d, generator=gen) * (d % 2)).to(odtype)  # zero, or what out held before
    want = to_np(start)
    oracle.sparse_linear_combination(d, rows, k, dbs, kb, coef.numpy(), to_np(I), to_np(V), want)
    out = start.cuda()
    if vdtype == odtype:
        smf.LCG(256, 1024, 51, d, rows, k, dbs, kb, coef.cuda(), I.cuda(), V.cuda(), out,
                int(vdtype == torch.bfloat16))
    else:  # the module's flag ties both types together: mixed types go through the C ABI
        Id, Vd, cd = I.cuda(), V.cuda(), coef.cuda()
        rc = hip_lib.lib.ma_sparse_linear_combination(
            d, rows, k, dbs, kb, hip_lib.dev_ptr(cd), hip_lib.dev_ptr(Id), hip_lib.dev_ptr(Vd),
            hip_lib.dtype_tag(Vd), hip_lib.dev_ptr(out), hip_lib.dtype_tag(out),
            hip_lib.stream_ptr())
        assert rc == 0
    got = to_np(out)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (bad[:5], got[bad[:5]], want[bad[:5]])


@pytest.fixture(scope="module")
def hip_lib():
    from ista_daslab_optimizers import _hip
    return _hip


@pytest.mark.parametrize("dense", [torch.bfloat16, torch.float32])
def test_copy_values_with_fp32_values(mods, dense):
    tools, _ = mods
    d, dbs = 20480 * 2 + 100, 20480
    I, V, k, kb = _window(3, d, dbs, 0.01, 1, torch.float32)
    pos = (torch.arange(k) // kb) * dbs + I[0].long()
    x = torch.randn(d, generator=torch.Generator().manual_seed(4)).to(dense)
    out = torch.zeros(k, dtype=torch.float32, device="cuda")
    tools.copy_values(d, k, dbs, kb, I[0].cuda(), x.cuda(), out, 1)
    assert torch.equal(out.cpu(), x[pos].float())
    back = torch.zeros(d, dtype=dense, device="cuda")
    tools.copy_values(d, k, dbs, kb, I[0].cuda(), V[0].cuda(), back, 0)
    want = torch.zeros(d, dtype=dense)
    want[pos] = V[0].to(dense)
    assert torch.equal(back.cpu(), want)


def test_rejected_arguments(hip_lib):
    import ctypes
    L = hip_lib.lib
    need = ctypes.c_int64()
    assert L.ma_sparse_scalar_products_workspace(61440, 8, 615, 20480, 205,
                                                 ctypes.byref(need)) == 0
    assert need.value == 3 * 8 * 4
    assert L.ma_sparse_scalar_products_workspace(61440, 5000, 615, 20480, 205,
                                                 ctypes.byref(need)) == -3
    assert L.ma_sparse_scalar_products_workspace(20480, 8, 615, 20480, 205,
                                                 ctypes.byref(need)) == -4
    x = torch.zeros(64, device="cuda")
    p = hip_lib.dev_ptr(x)
    # workspace too small
    assert L.ma_sparse_scalar_products(61440, 8, 615, 20480, 205, p, 0, p, p, 0, p, p, 16,
                                       None) == -1
    assert L.ma_sparse_linear_combination(61440, 8, 615, 40000, 205, p, p, p, 0, p, 0, None) == -2


def test_resnet50_sized_window_properties(mods, hip_lib):
    """At a ResNet-50-sized vector (25.6 M coordinates, 1248 top-k blocks, k = 1 %): a one-hot
    coefficient vector reproduces that row's scatter exactly; the scalar products of the rows
    with the scatter of row r give row r of a symmetric Gram matrix whose diagonal is the row's
    squared norm."""
    tools, smf = mods
    d, dbs, m = 25_557_032, 20480, 16
    lens, kbs, kb = _geometry(d, dbs, 0.01)
    k = sum(kbs)
    from ista_daslab_optimizers import _hip
    I = torch.zeros(m, k, dtype=torch.int16, device="cuda")
    V = torch.zeros(m, k, dtype=torch.bfloat16, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(0)
    for r in range(m):  # rows from the block top-k of random vectors, as the optimizer makes them
        x = torch.randn(d, generator=gen, device="cuda").to(torch.bfloat16)
        rc = _hip.lib.ma_block_topk(d, dbs, kb, kbs[-1], _hip.dev_ptr(x), _hip.dev_ptr(I[r]),
                                    _hip.dev_ptr(V[r]), 0, _hip.dtype_tag(x), _hip.stream_ptr())
        assert rc == 0
    gram = torch.zeros(m, m, dtype=torch.float32, device="cuda")
    for r in range(m):
        onehot = torch.zeros(m, dtype=torch.float32, device="cuda")
        onehot[r] = 1.0
        comb = torch.zeros(d, dtype=torch.bfloat16, device="cuda")
        smf.LCG(0, 0, 51, d, m, k, dbs, kb, onehot, I, V, comb, 1)
        scat = torch.zeros(d, dtype=torch.bfloat16, device="cuda")
        tools.copy_values(d, k, dbs, kb, I[r], V[r], scat, 0)
        assert torch.equal(comb, scat), r
        smf.SP(0, 0, 23, d, m, k, dbs, kb, scat, I, V, gram[r], 1)
    torch.cuda.synchronize()
    gram = gram.cpu().double()
    diag = (V.double() ** 2).sum(dim=1).cpu()
    assert torch.allclose(torch.diagonal(gram), diag, rtol=1e-5)
    scale = torch.sqrt(diag[:, None] * diag[None, :])
    assert torch.all((gram - gram.T).abs() <= 1e-5 * scale)
