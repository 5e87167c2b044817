"""ma_spanning_step_static (the entry point that allocates nothing: its scratch is a fixed
array in device memory) against ma_spanning_step (caller-provided workspace), through the C
ABI, bit for bit on everything the step writes: parameters, the residual left in the gradient
buffer, 4-bit codes, statistics and the window.  Two calls in a row, the second on a smaller
list, so that what the first call left in the array is seen not to matter.
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

KEYS = ("I", "V", "error", "min_vals", "max_vals")


def _prepared_state(sizes, m, q, alpha, steps):
    """Parameters, a fresh gradient and optimizer state after `steps` real steps."""
    from ista_daslab_optimizers import MicroAdam
    gen = torch.Generator(device="cuda").manual_seed(11)
    params = [torch.nn.Parameter((torch.randn(n, generator=gen, device="cuda") * 0.02)
                                 .to(torch.bfloat16)) for n in sizes]
    opt = MicroAdam(params, m=m, lr=1e-3, quant_block_size=q, k_init=0.01, alpha=alpha)
    for _ in range(steps):
        for p in params:
            p.grad = (torch.randn(p.numel(), generator=gen, device="cuda") * 1e-3).to(torch.bfloat16)
        opt.step()
    grads = [(torch.randn(p.numel(), generator=gen, device="cuda") * 1e-3).to(torch.bfloat16)
             for p in params]
    assert all(opt._fusable(p, opt.state[p]) == 2 for p in params)
    return opt, params, grads


def _copy_of(opt, params, grads, which):
    out = []
    for i in which:
        st = opt.state[params[i]]
        c = {k: st[k].clone() for k in KEYS}
        c.update(p=params[i].detach().clone(), g=grads[i].clone(), d=st["d"], k=st["k"],
                 index=st["index"])
        out.append(c)
    return out


def _call(entry, items, opt, alpha, t):
    from ista_daslab_optimizers import _hip
    arr = (_hip.MaTensor * len(items))()
    for a, c in zip(arr, items):
        a.p, a.g = c["p"].data_ptr(), c["g"].data_ptr()
        a.error, a.min_vals, a.max_vals = (c["error"].data_ptr(), c["min_vals"].data_ptr(),
                                           c["max_vals"].data_ptr())
        a.I, a.V = c["I"].data_ptr(), c["V"].data_ptr()
        a.d, a.k, a.lr, a.weight_decay, a.index = c["d"], c["k"], 1e-3, 0.01, c["index"]
    h = _hip.MaHyper(t, opt.m, _hip.MA_BF16, opt.quant_block_size, opt.d_block_size, opt.k_init,
                     opt.beta1, opt.beta2, opt.eps)
    if entry == "static":
        rc = _hip.lib.ma_spanning_step_static(arr, len(items), ctypes.byref(h), float(alpha),
                                              _hip.stream_ptr())
    else:
        need = _hip.lib.ma_spanning_step_workspace(arr, len(items), ctypes.byref(h))
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        rc = _hip.lib.ma_spanning_step(arr, len(items), ctypes.byref(h), float(alpha),
                                       ws.data_ptr(), ws.numel(), _hip.stream_ptr())
    torch.cuda.synchronize()
    return rc


@pytest.mark.parametrize("alpha", [0.5, 0.0])
def test_static_scratch_step_equals_workspace_step(alpha):
    sizes = [20480 * 7 + 77, 20480 * 3, 4096, 20480 * 12 + 4096, 2048]
    opt, params, grads = _prepared_state(sizes, 10, 100000, alpha, 3)
    # first the whole list, then a shorter list of shorter tensors
    for which in ([0, 1, 2, 3, 4], [2, 1]):
        want = _copy_of(opt, params, grads, which)
        got = _copy_of(opt, params, grads, which)
        assert _call("workspace", want, opt, alpha, 4) == 0
        assert _call("static", got, opt, alpha, 4) == 0
        for i, (a, b) in zip(which, zip(got, want)):
            # (not the gradient buffer: the step may or may not leave the residual there)
            for key in KEYS + ("p",):
                assert torch.equal(a[key].view(torch.uint8).view(-1),
                                   b[key].view(torch.uint8).view(-1)), (alpha, which, i, key)
        # the step did something: parameters moved and codes were written
        before = _copy_of(opt, params, grads, which)
        assert any(not torch.equal(a["p"], c["p"]) for a, c in zip(got, before))
        assert any(not torch.equal(a["error"], c["error"]) for a, c in zip(got, before))


def test_static_scratch_step_rejects_lists_beyond_its_array():
    """More top-k blocks than the array has room for: refused before anything is launched."""
    from ista_daslab_optimizers import _hip
    n_blocks = _hip.MA_STATIC_WORKSPACE_BYTES // 32 + 1
    t = (_hip.MaTensor * 1)()
    for f in ("p", "g", "error", "min_vals", "max_vals", "I", "V"):
        setattr(t[0], f, 0x10000)
    t[0].d = n_blocks * 512
    t[0].k = n_blocks * 6
    t[0].lr = 1e-3
    h = _hip.MaHyper(1, 4, _hip.MA_BF16, 512, 512, 0.01, 0.9, 0.999, 1e-8)
    rc = _hip.lib.ma_spanning_step_static(t, 1, ctypes.byref(h), 0.5, None)
    assert rc == _hip.MA_ERR_WORKSPACE
    assert "workspace" in _hip.error_string(rc)
