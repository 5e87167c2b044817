"""Golden fixtures (tests/golden/microadam_small.npz, written by tests/golden/make_golden.py):
the oracle must keep reproducing them, and so must the HIP path on the GPU."""
import os

import numpy as np
import pytest

from golden.make_golden import CASES

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "microadam_small.npz")
KEYS = ("I", "V", "error", "min_vals", "max_vals")


def _load():
    return np.load(FIX, allow_pickle=False)


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_reproduces_fixture(oracle, name):
    z = _load()
    sizes, dtype, m, q, k_init, alpha, wd, DB, steps = CASES[name]
    params = [z[f"{name}/p0/{i}"].copy() for i in range(len(sizes))]
    opt = oracle.OracleMicroAdam(params, m, 1e-3, q, k_init, alpha, weight_decay=wd, d_block_size=DB)
    for s in range(steps):
        opt.step([z[f"{name}/g/{s}/{i}"].copy() for i in range(len(sizes))])
    for i, p in enumerate(params):
        st = dict(opt.state[i])
        st["I"], st["V"] = oracle.canonical_window(st["I"], st["V"], st["k_block_size_many"])
        assert np.array_equal(p, z[f"{name}/p/{i}"])
        for key in KEYS:
            assert np.array_equal(np.asarray(st[key]).reshape(-1), z[f"{name}/{key}/{i}"].reshape(-1)), key
        assert st["index"] == int(z[f"{name}/index/{i}"])


@pytest.mark.gpu
@pytest.mark.parametrize("use_fused", [True, False], ids=["fused", "opbyop"])
@pytest.mark.parametrize("name", sorted(CASES))
def test_gpu_reproduces_fixture(oracle, name, use_fused):
    import torch
    from gpu_util import to_np, to_torch
    from ista_daslab_optimizers import MicroAdam
    z = _load()
    sizes, dtype, m, q, k_init, alpha, wd, DB, steps = CASES[name]
    params = [torch.nn.Parameter(to_torch(z[f"{name}/p0/{i}"])) for i in range(len(sizes))]
    opt = MicroAdam(params, m=m, lr=1e-3, quant_block_size=q, k_init=k_init, alpha=alpha,
                    weight_decay=wd)
    opt.d_block_size = DB
    opt.use_fused = use_fused
    for s in range(steps):
        for i, p in enumerate(params):
            p.grad = to_torch(z[f"{name}/g/{s}/{i}"])
        opt.step()
    for i, p in enumerate(params):
        st = opt.state[p]
        got = {key: to_np(st[key]) for key in KEYS}
        got["I"], got["V"] = oracle.canonical_window(got["I"], got["V"], st["k_block_size_many"])
        assert np.array_equal(to_np(p.data), z[f"{name}/p/{i}"]), "params"
        for key in KEYS:
            assert np.array_equal(got[key].reshape(-1), z[f"{name}/{key}/{i}"].reshape(-1)), key
        assert st["index"] == int(z[f"{name}/index/{i}"])


# ---- Sparse M-FAC's window kernels on the final windows of the cases above --------------------

from golden.make_golden import SPARSE_CASES  # noqa: E402


def _sparse_inputs(oracle, z, name):
    case, rows = SPARSE_CASES[name]
    sizes, dtype, m, q, k_init, alpha, wd, DB, steps = CASES[case]
    d = sizes[0]
    geo = oracle.geometry(d, DB, k_init, q)
    I, V = z[f"{case}/I/0"], z[f"{case}/V/0"]
    if dtype == "f32":
        V = oracle.bf16_to_f32(V)
    return d, rows, m, geo["k"], geo["d_block_size"], geo["k_block_size_many"], I, V


@pytest.mark.parametrize("name", sorted(SPARSE_CASES))
def test_oracle_reproduces_sparse_fixture(oracle, name):
    z = _load()
    d, rows, m, k, dbs, kb, I, V = _sparse_inputs(oracle, z, name)
    dots = np.zeros(m)
    oracle.sparse_scalar_products(d, rows, k, dbs, kb, z[f"{name}/g"], I, V, dots)
    assert np.array_equal(dots, z[f"{name}/dots"])
    comb = np.zeros(d, dtype=z[f"{name}/g"].dtype)
    oracle.sparse_linear_combination(d, rows, k, dbs, kb, z[f"{name}/coef"], I, V, comb)
    assert np.array_equal(comb, z[f"{name}/comb"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(SPARSE_CASES))
def test_gpu_reproduces_sparse_fixture(oracle, name):
    """Linear combination bit for bit; scalar products within 2e-6 of the sum of the absolute
    terms (the order of the device's fp32 sum is its own)."""
    import torch
    import ista_daslab_cuda_sparse_mfac as smf
    from gpu_util import to_np, to_torch
    z = _load()
    d, rows, m, k, dbs, kb, I, V = _sparse_inputs(oracle, z, name)
    g, Id, Vd = to_torch(z[f"{name}/g"]), torch.from_numpy(I.copy()).cuda(), to_torch(V)
    bf16 = int(g.dtype == torch.bfloat16)
    dots = torch.zeros(m, dtype=torch.float32, device="cuda")
    smf.SP(0, 0, 23, d, rows, k, dbs, kb, g, Id, Vd, dots, bf16)
    pos = (torch.arange(k) // kb) * dbs + torch.from_numpy(I.astype(np.int64))
    mass = (Vd.cpu().double().abs() * g.cpu().double()[pos].abs()).sum(dim=1).numpy()
    assert np.all(np.abs(dots.cpu().numpy() - z[f"{name}/dots"]) <= 2e-6 * mass + 1e-30)
    comb = torch.zeros(d, dtype=g.dtype, device="cuda")
    smf.LCG(0, 0, 51, d, rows, k, dbs, kb, torch.from_numpy(z[f"{name}/coef"]).cuda(), Id, Vd,
            comb, bf16)
    assert np.array_equal(to_np(comb), z[f"{name}/comb"])
