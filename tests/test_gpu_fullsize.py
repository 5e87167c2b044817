"""Full-size checks on the GPU, at the tensor shapes of the Llama-2-7B, outlier-1.3B and
Llama-3-8B lists,
through properties that do not need the CPU oracle at that size:

  * the fused kernel and the op-by-op kernels (two independent implementations of selection,
    statistics, quantisation and update) end in bit-identical parameters and state;
  * every block row of the window holds distinct in-range indices, and what it holds really is
    the top-k: no unselected magnitude exceeds the smallest selected one;
  * error feedback round trip: Qinv(e_new) reproduces the residual within half a step
    ((1 - alpha) x the residual within a step when alpha > 0);
  * with alpha == 0, parameters move only at coordinates the window names.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _canon(I, V, k_many):
    blk = torch.arange(I.shape[1], device=I.device) // k_many
    key = blk[None, :].long() * 65536 + I.long()
    order = torch.argsort(key, dim=1, stable=True)
    return torch.gather(I, 1, order), torch.gather(V.view(torch.int16), 1, order)


def _grads(shape, kind, step, dtype):
    g = torch.Generator(device="cuda").manual_seed(1000 + step)
    if kind == "normal":
        return (torch.randn(shape, generator=g, device="cuda") * 1e-3).to(dtype)
    # Student-t(3) scaled by 1e-3 with 1 % outlier rows x100 (the stress recipe)
    z = torch.randn(shape, generator=g, device="cuda")
    chi = (torch.randn((3,) + tuple(shape), generator=g, device="cuda") ** 2).sum(0) / 3
    t = z / chi.sqrt() * 1e-3
    if len(shape) == 2:
        rows = torch.rand(shape[0], generator=torch.Generator(device="cuda").manual_seed(7),
                          device="cuda") < 0.01
        t[rows] *= 100
    return t.to(dtype)


CASES = [
    # shapes, m, k_init, q, grad kind, steps, dtype
    ([(32000, 4096), (11008, 4096), (4096, 4096), (4096,)], 10, 0.01, 64, "normal", 12,
     torch.bfloat16),
    # the outlier list's shapes, past the point where its window of 20 rows is full and wraps
    ([(50304, 2048), (2048, 8192), (2048, 6144), (2048, 2048), (2048,)], 20, 0.05, 32, "outlier",
     23, torch.bfloat16),
    ([(11008, 4096), (4096,)], 10, 0.01, 64, "normal", 12, torch.float32),
]


def _routes_agree(oa, ob, pa, pb, step):
    for p, p2 in zip(pa, pb):
        sa, sb = oa.state[p], ob.state[p2]
        assert sa["index"] == sb["index"]
        assert torch.equal(p.data, p2.data), f"step {step}: parameters differ between routes"
        for key in ("error", "min_vals", "max_vals"):
            assert torch.equal(sa[key], sb[key]), (step, key)
        km = sa["k_block_size_many"]
        Ia, Va = _canon(sa["I"], sa["V"], km)
        Ib, Vb = _canon(sb["I"], sb["V"], km)
        assert torch.equal(Ia, Ib) and torch.equal(Va, Vb), (step, "window")


def _accumulator(ext, st, g, q):
    """a = g + Qinv(e_prev), from the op-by-op kernel."""
    a = g.detach().clone().view(-1)
    if len(st):
        ext.asymm_block_quant_inv(a.numel(), q, st["error"], st["min_vals"], st["max_vals"], a, 1.0)
    return a


def _check_properties(ext, st, p, a, p0, step, m, q, alpha):
    """What one step must have done to one tensor, given its accumulator a and its parameters
    before the step: the row written is the block-wise top-k of |a| with V == a[I]; the stored
    error feedback reproduces (1 - alpha) x the residual; with alpha == 0 the parameters moved
    only at coordinates the window names."""
    km, dbs, k = st["k_block_size_many"], st["d_block_size"], st["k"]
    row = (st["index"] - 1) % m
    idx = st["I"][row].long()
    assert int(idx.min()) >= 0
    pos = (torch.arange(k, device="cuda") // km) * dbs + idx
    assert int(pos.max()) < a.numel()
    assert torch.unique(pos).numel() == k, "duplicate index in a block row"
    mag = a.float().abs()
    assert torch.equal(st["V"][row], a[pos].to(torch.bfloat16)), "window values are not a[I]"
    sel = torch.zeros_like(mag, dtype=torch.bool)
    sel[pos] = True
    nblk = (a.numel() + dbs - 1) // dbs
    pad = nblk * dbs - a.numel()
    mag_p = torch.nn.functional.pad(mag, (0, pad), value=-1.0).view(nblk, dbs)
    sel_p = torch.nn.functional.pad(sel, (0, pad), value=False).view(nblk, dbs)
    smallest_kept = torch.where(sel_p, mag_p, torch.full_like(mag_p, float("inf"))).amin(1)
    largest_left = torch.where(sel_p, torch.full_like(mag_p, -1.0), mag_p).amax(1)
    assert bool((smallest_kept >= largest_left).all()), "a larger magnitude was left out"
    del mag_p, sel_p, sel, mag
    # error feedback round trip
    resid = a.clone()
    resid[pos] = 0
    deq = torch.zeros_like(a)
    ext.asymm_block_quant_inv(a.numel(), q, st["error"], st["min_vals"], st["max_vals"], deq, 1.0)
    nq = (a.numel() + q - 1) // q
    u = (st["max_vals"][:nq].float() - st["min_vals"][:nq].float()) / 15
    u = u.repeat_interleave(q)[: a.numel()]
    if alpha == 0:
        # half a quantisation step, plus the bf16 rounding of the dequantised value itself
        tol = u / 2 + deq.float().abs() * 2.0 ** -8 + 1e-12
    else:
        # the stored codes are of r2 = (1 - alpha) * Qinv(Q(residual)): half a step of each of
        # the two quantisations (the first one's step is the second's / (1 - alpha)), and the
        # roundings of r2 and of the dequantised value
        tol = u * 1.01 + deq.float().abs() * 2.0 ** -7 + 1e-12
    want = resid.float() * (1.0 - alpha)
    assert bool(((deq.float() - want).abs() <= tol).all()), "EF round trip"
    del resid, deq, u, tol, want
    if alpha == 0:  # parameters move only where the window points
        live = min(step + 1, m)
        touched = torch.zeros(a.numel(), dtype=torch.bool, device="cuda")
        for r in range(live):
            touched[(torch.arange(k, device="cuda") // km) * dbs + st["I"][r].long()] = True
        moved = (p.data.view(-1) != p0.view(-1))
        assert not bool((moved & ~touched).any())


@pytest.mark.parametrize("shapes,m,k_init,q,kind,steps,dtype", CASES)
def test_fused_and_opbyop_agree_and_select_topk(shapes, m, k_init, q, kind, steps, dtype):
    from ista_daslab_optimizers import MicroAdam
    import ista_daslab_cuda_micro_adam as ext
    torch.manual_seed(0)
    pa = [torch.nn.Parameter((torch.randn(s, device="cuda") * 0.02).to(dtype)) for s in shapes]
    pb = [torch.nn.Parameter(p.detach().clone()) for p in pa]
    oa = MicroAdam(pa, m=m, lr=1e-3, quant_block_size=q, k_init=k_init)
    ob = MicroAdam(pb, m=m, lr=1e-3, quant_block_size=q, k_init=k_init)
    ob.use_fused = False
    # the properties at the first steps, around the step that fills the window, and at the end
    check_at = {0, 1, 2, m - 2, m - 1, m, steps - 2, steps - 1}
    for step in range(steps):
        grads = [_grads(s, kind, step * 10 + i, dtype) for i, s in enumerate(shapes)]
        check = step in check_at
        before = [p.detach().clone() for p in pa] if check else None
        acc = [_accumulator(ext, oa.state.get(p, {}), g, q) for p, g in zip(pa, grads)] if check else None
        for p, p2, g in zip(pa, pb, grads):
            p.grad, p2.grad = g.clone(), g.clone()
        oa.step()
        ob.step()
        assert all(oa._fusable(p, oa.state[p]) == 1 for p in pa)
        _routes_agree(oa, ob, pa, pb, step)
        if check:
            for p, a, p0 in zip(pa, acc, before):
                _check_properties(ext, oa.state[p], p, a, p0, step, m, q, 0.0)


def test_spanning_and_opbyop_agree_at_llama3_shapes():
    """The Llama-3-8B list's shapes and hyper-parameters: alpha = 0.5 with quantisation blocks of
    100000 elements, which straddle the 20480-element top-k blocks.  The two-pass fused route
    and the op-by-op kernels, which form the statistics in different ways, end in bit-identical
    parameters and state, and the step has the properties listed at the top of the file (the
    embedding's 25651 top-k blocks and 5254 quantisation blocks included)."""
    from ista_daslab_optimizers import MicroAdam
    import ista_daslab_cuda_micro_adam as ext
    shapes = [(128256, 4096), (14336, 4096), (4096, 4096), (1024, 4096), (4096,)]
    dtype, m, q, alpha, steps = torch.bfloat16, 10, 100000, 0.5, 12
    torch.manual_seed(0)
    pa = [torch.nn.Parameter((torch.randn(s, device="cuda") * 0.02).to(dtype)) for s in shapes]
    pb = [torch.nn.Parameter(p.detach().clone()) for p in pa]
    kw = dict(m=m, lr=1e-3, quant_block_size=q, k_init=0.01, alpha=alpha)
    oa, ob = MicroAdam(pa, **kw), MicroAdam(pb, **kw)
    ob.use_fused = False
    check_at = {0, 1, m - 1, m, steps - 1}
    for step in range(steps):
        grads = [_grads(s, "normal", step * 10 + i, dtype) for i, s in enumerate(shapes)]
        check = step in check_at
        acc = [_accumulator(ext, oa.state.get(p, {}), g, q) for p, g in zip(pa, grads)] if check else None
        for p, p2, g in zip(pa, pb, grads):
            p.grad, p2.grad = g.clone(), g.clone()
        oa.step()
        ob.step()
        assert all(oa._fusable(p, oa.state[p]) == 2 for p in pa)
        _routes_agree(oa, ob, pa, pb, step)
        if check:
            for p, a in zip(pa, acc):
                _check_properties(ext, oa.state[p], p, a, None, step, m, q, alpha)
