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
