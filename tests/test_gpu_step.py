"""GPU parity of the whole optimizer step, through the MicroAdam class, against the oracle.

Both routes of the class (the fused kernel and the op-by-op sequence) must reproduce the
oracle's state bit for bit: window indices and values, 4-bit error-feedback codes, bf16
min/max statistics, and here also the parameters themselves (the kernels use the same
unfused fp32 arithmetic as the oracle, so the stated 1e-3 / 1e-5 tolerance is met with
zero difference; the tolerance check is kept as the documented bar).
"""
import functools

import numpy as np
import pytest
import torch

from gpu_util import assert_state_equal, to_np

pytestmark = pytest.mark.gpu

REL_TOL = {torch.bfloat16: 1e-3, torch.float32: 1e-5}


def _run(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps, use_fused, grad_scale=1e-2,
         zero_step=None, lr=1e-3, seed=0, expect_route=None):
    from ista_daslab_optimizers import MicroAdam
    gen = torch.Generator().manual_seed(seed)
    cpu_params = [(torch.randn(n, generator=gen) * 0.02).to(dtype) for n in sizes]
    oparams = [to_np(p) for p in cpu_params]
    oref = oracle.OracleMicroAdam(oparams, m, lr, q, k_init, alpha, weight_decay=wd, d_block_size=DB)
    gparams = [torch.nn.Parameter(p.clone().cuda()) for p in cpu_params]
    opt = MicroAdam(gparams, m=m, lr=lr, quant_block_size=q, k_init=k_init, alpha=alpha,
                    weight_decay=wd)
    opt.d_block_size = DB
    opt.use_fused = use_fused
    for s in range(steps):
        grads = [(torch.randn(n, generator=gen) * grad_scale).to(dtype) for n in sizes]
        if zero_step is not None and s == zero_step:
            grads[0].zero_()
        for p, g in zip(gparams, grads):
            p.grad = g.clone().cuda()
        opt.step()
        oref.step([to_np(g) for g in grads])
        for i, p in enumerate(gparams):
            ctx = f"step {s + 1} tensor {i} (d={sizes[i]})"
            assert_state_equal(opt.state[p], oref.state[i], ctx)
            if alpha == -2:  # st['quant_err'] = a - Qinv(e_new), rewritten by every step
                assert np.array_equal(to_np(opt.state[p]["quant_err"]).reshape(-1),
                                      oref.state[i]["quant_err"]), f"{ctx}: quant_err"
            got, want = to_np(p.data), oparams[i]
            if not np.array_equal(got, want):
                gf = oracle.bf16_to_f32(got) if got.dtype == np.uint16 else got
                wf = oracle.bf16_to_f32(want) if want.dtype == np.uint16 else want
                rel = np.abs(gf - wf).max() / max(np.abs(wf).max(), 1e-30)
                raise AssertionError(f"{ctx}: parameters differ at {(got != want).sum()} entries, "
                                     f"max rel {rel:.3e} (bar {REL_TOL[dtype]})")
    if expect_route is not None:
        fused_now = [opt._fusable(p, opt.state[p]) and use_fused for p in gparams
                     if p.grad is not None]
        assert all(fused_now) == expect_route, fused_now
    return opt


CASES = [
    # sizes, dtype, m, q, k_init, alpha, wd, DB, steps
    ([3000, 257, 64, 1024], torch.bfloat16, 4, 64, 0.01, 0.0, 0.0, 1024, 9),
    ([5000], torch.float32, 3, 64, 0.02, 0.0, 0.0, 2048, 7),
    ([2500, 130], torch.bfloat16, 5, 32, 0.05, 0.0, 0.1, 512, 8),
    ([20480 * 2 + 4096, 768, 4096], torch.bfloat16, 10, 64, 0.01, 0.0, 0.0, 20480, 12),
    ([20480 + 4096], torch.float32, 10, 64, 0.01, 0.0, 0.01, 20480, 12),
    ([32768 + 1000], torch.bfloat16, 3, 128, 0.01, 0.0, 0.0, 32768, 5),
    ([10240 * 2 + 8], torch.bfloat16, 3, 8, 0.01, 0.0, 0.0, 10240, 5),
    ([1001, 777], torch.bfloat16, 3, 64, 0.03, 0.0, 0.0, 20480, 5),   # odd d: partial chunks
    # windows too large for the one-pass stage (20 rows of 5 %): the step in two launches, the
    # rows' chunk cuts cached; with weight decay and a tensor of exactly one block; more rows;
    # fp32 data (the general selection, fp32 parameters in the window kernel)
    ([20480 * 2 + 8192], torch.bfloat16, 20, 32, 0.05, 0.0, 0.0, 20480, 23),
    ([20480 * 2 + 4096, 20480], torch.bfloat16, 20, 64, 0.05, 0.0, 0.01, 20480, 22),
    ([20480 + 8192], torch.bfloat16, 24, 32, 0.05, 0.0, 0.0, 20480, 26),
    ([20480 * 2 + 8192], torch.float32, 20, 32, 0.05, 0.0, 0.0, 20480, 22),
    # more rows than the one-pass stage takes, but short block rows (1 %), which the fast
    # selections do not list by coordinate: two launches, the window kernel's general form
    ([20480 * 2 + 8192, 4096], torch.bfloat16, 18, 64, 0.01, 0.0, 0.0, 20480, 21),
    # a fifth of every block selected: a row has about 100 entries per 512 coordinates, more
    # than the window kernel's 64 lanes take in one go
    ([20480 * 2 + 4096], torch.bfloat16, 4, 64, 0.2, 0.0, 0.0, 20480, 7),
    # quantisation blocks longer than the 512 elements a wave holds per chunk
    ([20480 * 2 + 4096, 3000, 12288], torch.bfloat16, 4, 1024, 0.01, 0.0, 0.0, 20480, 6),
    ([20480 + 5000], torch.bfloat16, 10, 4096, 0.01, 0.0, 0.01, 20480, 12),
    ([20480 + 2048 + 77, 4096], torch.float32, 3, 2048, 0.01, 0.0, 0.0, 20480, 5),
    ([32768 + 9000], torch.bfloat16, 3, 4096, 0.01, 0.0, 0.0, 32768, 5),
    # more tensors of one size class than one launch takes (160): two launches
    ([96 + 8 * (i % 5) for i in range(190)] + [3000], torch.bfloat16, 3, 8, 0.05, 0.0, 0.0, 1024, 4),
]


@pytest.mark.parametrize("use_fused", [True, False], ids=["fused", "opbyop"])
@pytest.mark.parametrize("sizes,dtype,m,q,k_init,alpha,wd,DB,steps", CASES)
def test_step_matches_oracle(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps, use_fused):
    _run(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps, use_fused, zero_step=2,
         expect_route=use_fused)


GENERAL_CASES = [
    # alpha > 0, odd quantisation blocks, d < q: only the op-by-op route applies
    ([4100, 33], torch.bfloat16, 3, 1000, 0.01, 0.5, 0.0, 1024, 7),
    ([999], torch.float32, 2, 100, 0.03, 0.25, 0.01, 400, 5),
    ([20480 * 3 + 77], torch.bfloat16, 4, 100001, 0.01, 0.5, 0.0, 20480, 6),
    ([50, 20], torch.bfloat16, 3, 60, 0.1, 0.0, 0.0, 20480, 4),
    # alpha == -2 with quantisation blocks that the one-pass kernels do not take
    ([4100, 33], torch.bfloat16, 3, 1000, 0.01, -2, 0.0, 1024, 5),
]


@pytest.mark.parametrize("sizes,dtype,m,q,k_init,alpha,wd,DB,steps", GENERAL_CASES)
def test_step_general_route(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps):
    _run(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps, True, expect_route=False)


QUANT_ERR_CASES = [
    # alpha == -2: the quantisation error goes straight into the parameters
    # (micro_adam.py:238-273), inside the one-pass kernels
    ([20480 + 4096, 300], torch.bfloat16, 4, 64, 0.01, -2, 0.0, 20480, 6),
    ([3000], torch.float32, 3, 64, 0.02, -2, 0.05, 1024, 5),
    ([20480 * 3, 1001], torch.bfloat16, 10, 64, 0.01, -2, 0.01, 20480, 12),
    ([20480 * 2 + 8192], torch.bfloat16, 20, 32, 0.05, -2, 0.0, 20480, 22),
    ([20480 + 77], torch.float32, 5, 32, 0.01, -2, 0.0, 20480, 7),
    ([20480 * 2 + 1000], torch.bfloat16, 4, 2048, 0.01, -2, 0.0, 20480, 6),
]


@pytest.mark.parametrize("use_fused", [True, False], ids=["fused", "opbyop"])
@pytest.mark.parametrize("sizes,dtype,m,q,k_init,alpha,wd,DB,steps", QUANT_ERR_CASES)
def test_step_quant_err_route(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps, use_fused):
    opt = _run(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps, use_fused, zero_step=2,
               expect_route=use_fused)
    # micro_adam.py:67-68; _run has compared it with the oracle's after every step
    assert all(st["quant_err"].any() for st in opt.state.values())


SPANNING_CASES = [
    # quantisation blocks at least as long as the top-k blocks: two-pass route
    ([20480 * 5 + 77], torch.bfloat16, 10, 100000, 0.01, 0.5, 0.0, 20480, 12),
    ([20480 * 12 + 4096, 4096, 1000], torch.bfloat16, 4, 24576, 0.01, 0.3, 0.01, 20480, 8),
    ([5000, 3000], torch.float32, 3, 2048, 0.02, 0.25, 0.0, 1024, 6),
    ([40000], torch.bfloat16, 3, 20480, 0.01, 0.9, 0.0, 20480, 5),
    ([512 * 9 + 100], torch.bfloat16, 3, 520, 0.02, 0.5, 0.0, 512, 6),
    # alpha == 0 with long quantisation blocks (the reference's documented quant_block_size)
    ([20480 * 5 + 77, 4096], torch.bfloat16, 10, 100000, 0.01, 0.0, 0.0, 20480, 12),
    ([5000, 3000], torch.float32, 3, 2048, 0.02, 0.0, 0.01, 1024, 6),
    ([50, 20], torch.bfloat16, 3, 64, 0.1, 0.0, 0.0, 20480, 4),       # d < q
]


@pytest.mark.parametrize("use_fused", [True, False], ids=["spanning", "opbyop"])
@pytest.mark.parametrize("sizes,dtype,m,q,k_init,alpha,wd,DB,steps", SPANNING_CASES)
def test_step_spanning_route(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps, use_fused):
    _run(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps, use_fused, zero_step=2,
         expect_route=use_fused)


FUSED_DENSIFIED_CASES = [
    # 0 < alpha < 1 with quantisation blocks inside the top-k blocks: one pass
    ([20480 * 2 + 4096, 768, 4096], torch.bfloat16, 10, 64, 0.01, 0.5, 0.0, 20480, 12),
    ([3000, 257, 64, 1024], torch.bfloat16, 4, 64, 0.01, 0.25, 0.1, 1024, 9),
    ([5000], torch.float32, 3, 64, 0.02, 0.7, 0.0, 2048, 7),
    ([20480 + 4096], torch.float32, 10, 32, 0.01, 0.1, 0.01, 20480, 12),
    ([1001, 777], torch.bfloat16, 3, 64, 0.03, 0.5, 0.0, 20480, 5),   # odd d: partial chunks
    # quantisation blocks longer than the 512 elements a wave holds per chunk
    ([20480 * 2 + 4096, 3000], torch.bfloat16, 3, 1024, 0.01, 0.5, 0.0, 20480, 4),
    ([20480 + 5000], torch.float32, 4, 4096, 0.01, 0.3, 0.01, 20480, 6),
    ([32768 + 9000], torch.bfloat16, 3, 2048, 0.01, 0.7, 0.0, 32768, 5),
]


@pytest.mark.parametrize("use_fused", [True, False], ids=["fused", "opbyop"])
@pytest.mark.parametrize("sizes,dtype,m,q,k_init,alpha,wd,DB,steps", FUSED_DENSIFIED_CASES)
def test_step_fused_densified_route(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps,
                                    use_fused):
    _run(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB, steps, use_fused, zero_step=2,
         expect_route=use_fused)


@pytest.mark.parametrize("use_fused", [True, False], ids=["fused", "opbyop"])
@pytest.mark.parametrize("scale", [1e-36, 3e-38, 1e-39])
def test_denormal_scale_gradients(oracle, scale, use_fused):
    """Gradients so small that quantisation steps and window values are fp32 / bf16 denormals:
    no flush to zero anywhere, and codes stay inside [0, 15] when the step (max - min) / 15
    is rounded coarsely."""
    _run(oracle, [20480 + 4096], torch.bfloat16, 3, 64, 0.01, 0.0, 0.0, 20480, 5, use_fused,
         grad_scale=scale)


@pytest.mark.parametrize("use_fused", [True, False], ids=["fused", "opbyop"])
def test_config1_plumbing(oracle, use_fused):
    """The plumbing configuration: one flat fp32 parameter, d = 1,048,576, N(0,1) gradients,
    m=10, k=1 %, q=64, hardware block size; run on to 100 steps (the configuration asks for 20;
    the fp32 tolerance is stated after 100), state and parameters compared after every step."""
    opt = _run(oracle, [1048576], torch.float32, 10, 64, 0.01, 0.0, 0.0, 20480, 100, use_fused,
               grad_scale=1.0, expect_route=use_fused)
    assert opt.d_block_size == 20480 and opt.steps == 100


def test_outlier_gradients(oracle):
    """Heavy-tailed gradients with outlier rows (the stress configuration's recipe, small)."""
    from ista_daslab_optimizers import MicroAdam
    gen = torch.Generator().manual_seed(3)
    rows, cols = 64, 2048
    p0 = (torch.randn(rows * cols, generator=gen) * 0.02).to(torch.bfloat16)
    hot = torch.rand(rows, generator=gen) < 0.05
    oparams = [to_np(p0)]
    oref = oracle.OracleMicroAdam(oparams, 20, 1e-3, 32, 0.05, 0, d_block_size=20480)
    gp = torch.nn.Parameter(p0.clone().cuda())
    opt = MicroAdam([gp], m=20, lr=1e-3, quant_block_size=32, k_init=0.05)
    dist = torch.distributions.StudentT(3.0)
    for s in range(6):
        torch.manual_seed(100 + s)
        g = dist.sample((rows, cols)) * 1e-3
        g[hot] *= 100
        g = g.to(torch.bfloat16).view(-1)
        gp.grad = g.clone().cuda()
        opt.step()
        oref.step([to_np(g)])
        assert_state_equal(opt.state[gp], oref.state[0], f"step {s + 1}")
        assert np.array_equal(to_np(gp.data), oparams[0])


def test_lr_schedule_none_grads_and_closure(oracle):
    """group['lr'] is re-read every step, parameters without a gradient are skipped, and the
    closure's loss is returned (micro_adam.py:102-105, 121, 125-126)."""
    from ista_daslab_optimizers import MicroAdam
    gen = torch.Generator().manual_seed(5)
    sizes = [4096, 2048]
    cpu = [(torch.randn(n, generator=gen) * 0.02).to(torch.bfloat16) for n in sizes]
    oparams = [to_np(p) for p in cpu]
    oref = oracle.OracleMicroAdam(oparams, 4, 1e-3, 64, 0.01, 0, d_block_size=20480)
    gparams = [torch.nn.Parameter(p.clone().cuda()) for p in cpu]
    opt = MicroAdam(gparams, m=4, lr=1e-3, quant_block_size=64)
    for s in range(6):
        lr = 1e-3 * (s + 1)
        opt.param_groups[0]["lr"] = lr
        grads = [(torch.randn(n, generator=gen) * 1e-2).to(torch.bfloat16) for n in sizes]
        if s % 2:
            grads[1] = None
        for p, g in zip(gparams, grads):
            p.grad = None if g is None else g.clone().cuda()
        loss = opt.step(closure=lambda: torch.tensor(1.5 + s))
        assert float(loss) == 1.5 + s
        oref.step([None if g is None else to_np(g) for g in grads], lr=lr)
        for i, p in enumerate(gparams):
            if oref.state[i] is not None:
                assert_state_equal(opt.state[p], oref.state[i], f"step {s + 1} tensor {i}")
            assert np.array_equal(to_np(p.data), oparams[i])


def test_logging_with_mixed_types_and_missing_gradients(oracle):
    """One list holding bf16 and fp32 tensors of all block classes, and on some logging steps a
    tensor without a gradient: the step is then several library calls (one per route and element
    type), whose kernels add their shares to the same six sums (micro_adam.py:121, 125-136,
    328, 330)."""
    from ista_daslab_optimizers import MicroAdam
    gen = torch.Generator().manual_seed(21)
    spec = [(20480 * 2 + 300, torch.bfloat16), (768, torch.bfloat16), (20480 + 8, torch.float32),
            (3000, torch.float32), (10000, torch.bfloat16)]
    cpu = [(torch.randn(n, generator=gen) * 0.02).to(dt) for n, dt in spec]
    oparams = [to_np(p) for p in cpu]
    oref = oracle.OracleMicroAdam(oparams, 4, 1e-3, 64, 0.01, 0, weight_decay=0.01)
    gparams = [torch.nn.Parameter(p.clone().cuda()) for p in cpu]
    opt = MicroAdam(gparams, m=4, lr=1e-3, quant_block_size=64, weight_decay=0.01)
    opt.log_interval = 2
    opt._logging_active = lambda: True
    logged = []
    opt._log = lambda *a: logged.append([float(x) for x in a[:6]])
    calls = []
    inner = opt._fused_step
    opt._fused_step = lambda route, dtype, entries, sums=None: (
        calls.append((opt.steps, dtype, len(entries), sums is not None)),
        inner(route, dtype, entries, sums))
    wanted = []
    for s in range(6):
        grads = [(torch.randn(n, generator=gen) * 1e-2).to(dt) for n, dt in spec]
        if s in (1, 4):
            grads[2] = None     # step 2 is a logging step, step 5 is not
        for p, g in zip(gparams, grads):
            p.grad = None if g is None else g.clone().cuda()
        opt.step()
        out = oref.step([None if g is None else to_np(g) for g in grads], metrics=(s + 1) % 2 == 0)
        if out is not None:
            wanted.append(out)
        for i, p in enumerate(gparams):
            if oref.state[i] is not None:
                assert_state_equal(opt.state[p], oref.state[i], f"step {s + 1} tensor {i}")
            assert np.array_equal(to_np(p.data), oparams[i]), f"step {s + 1} tensor {i}"
    # two calls per step (bf16, fp32), with sums exactly on the logging steps
    assert [c for c in calls if c[0] == 2] == [(2, torch.bfloat16, 3, True), (2, torch.float32, 1, True)]
    assert [c for c in calls if c[0] == 3] == [(3, torch.bfloat16, 3, False), (3, torch.float32, 2, False)]
    assert len(logged) == 3 == len(wanted)
    keys = ("norm_qe", "norm_g", "norm_u", "norm_e", "sparsity_u", "sparsity_qe")
    for got, want in zip(logged, wanted):
        for key, value in zip(keys, got):
            if key.startswith("sparsity"):
                assert value == want[key], (key, value, want[key])
            else:
                assert value == pytest.approx(want[key], rel=1e-5, abs=0), (key, value, want[key])


def test_state_layout_and_checkpoint_roundtrip():
    """State keys, dtypes and shapes as micro_adam.py:61-94; state_dict round trip, including
    the re-typing load_state_dict applies to floating-point state."""
    from ista_daslab_optimizers import MicroAdam
    torch.manual_seed(0)
    p = torch.nn.Parameter(torch.randn(20480 + 4096, device="cuda") * 0.02)
    opt = MicroAdam([p], m=10, lr=1e-3, quant_block_size=64)
    for _ in range(3):
        p.grad = torch.randn_like(p) * 1e-2
        opt.step()
    st = opt.state[p]
    assert st["I"].dtype == torch.int16 and st["I"].shape == (10, 205 + 41)
    assert st["V"].dtype == torch.bfloat16 and st["V"].shape == (10, 246)
    assert st["error"].dtype == torch.uint8 and st["error"].numel() == (20480 + 4096) // 2
    assert st["min_vals"].dtype == torch.bfloat16 and st["min_vals"].numel() == 384 + 1
    assert (st["index"], st["k"], st["d_block_size"], st["k_block_size_many"],
            st["k_block_size_few"], st["d_index_topk"]) == (3, 246, 20480, 205, 41, 20480)
    sd = opt.state_dict()
    p2 = torch.nn.Parameter(p.detach().clone())
    opt2 = MicroAdam([p2], m=10, lr=1e-3, quant_block_size=64)
    opt2.load_state_dict(sd)
    assert opt2.steps == opt.steps  # the reference loses the counter on resume (micro_adam.py:35)
    g = torch.randn_like(p) * 1e-2
    p.grad, p2.grad = g.clone(), g.clone()
    opt.step()
    opt2.step()
    assert opt2.state[p2]["V"].dtype == torch.bfloat16
    assert torch.equal(p.data, p2.data)
    for key in ("I", "V", "error", "min_vals", "max_vals"):
        assert torch.equal(opt.state[p][key], opt2.state[p2][key]), key
    # a framework that re-types the state (every tensor cast to the parameter's dtype) is
    # repaired on the next step, as the reference does for st['I']
    st2 = opt2.state[p2]
    for key in ("I", "V", "error", "min_vals", "max_vals"):
        st2[key] = st2[key].to(torch.float32)
    p.grad, p2.grad = g.clone(), g.clone()
    opt.step()
    opt2.step()
    assert st2["I"].dtype == torch.int16 and st2["error"].dtype == torch.uint8
    assert torch.equal(p.data, p2.data)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_checkpoint_through_a_file(oracle, tmp_path, dtype):
    """torch.save -> torch.load(weights_only=True) -> load_state_dict into a fresh optimizer,
    mid-run and after the ring has wrapped: the resumed run continues bit for bit like the
    uninterrupted one and like the oracle (which never stopped), on the fused route."""
    from ista_daslab_optimizers import MicroAdam
    sizes, m = [20480 * 2 + 4096, 768], 4
    gen = torch.Generator().manual_seed(5)
    cpu_params = [(torch.randn(n, generator=gen) * 0.02).to(dtype) for n in sizes]
    oparams = [to_np(p) for p in cpu_params]
    oref = oracle.OracleMicroAdam(oparams, m, 1e-3, 64, 0.01, 0, weight_decay=0.01)
    params = [torch.nn.Parameter(p.clone().cuda()) for p in cpu_params]
    opt = MicroAdam(params, m=m, lr=1e-3, quant_block_size=64, weight_decay=0.01)
    for s in range(11):
        if s in (2, 7):  # before and after the window is full
            path = tmp_path / f"ckpt{s}.pt"
            torch.save({"opt": opt.state_dict(), "params": [p.data for p in params]}, path)
            del opt, params
            blob = torch.load(path, map_location="cuda", weights_only=True)
            params = [torch.nn.Parameter(t.clone()) for t in blob["params"]]
            opt = MicroAdam(params, m=m, lr=1e-3, quant_block_size=64, weight_decay=0.01)
            opt.load_state_dict(blob["opt"])
            assert opt.steps == s
            for p in params:
                st = opt.state[p]
                assert st["I"].dtype == torch.int16 and st["error"].dtype == torch.uint8
                assert st["V"].dtype == st["min_vals"].dtype == torch.bfloat16
                assert st["index"] == s % m
        grads = [(torch.randn(n, generator=gen) * 1e-2).to(dtype) for n in sizes]
        for p, g in zip(params, grads):
            p.grad = g.clone().cuda()
        opt.step()
        assert all(opt._fusable(p, opt.state[p]) == 1 for p in params)
        oref.step([to_np(g) for g in grads])
        for i, p in enumerate(params):
            assert_state_equal(opt.state[p], oref.state[i], f"step {s + 1} tensor {i}")
            assert np.array_equal(to_np(p.data), oparams[i]), f"step {s + 1} tensor {i}"


def test_checkpoint_made_for_another_block_size(oracle):
    """State whose geometry was derived from another device's top-k block size (the reference
    sizes d_block_size from the shared memory of the GPU it runs on, micro_adam.py:43-44): the
    fused kernels would derive a different geometry from this optimizer's own, so such tensors
    take the op-by-op route, which reads the stored geometry, and still match an oracle that
    runs with the checkpoint's block size."""
    from ista_daslab_optimizers import MicroAdam
    n, m, foreign = 20480 * 2 + 4096, 4, 12288
    gen = torch.Generator().manual_seed(6)
    p0 = (torch.randn(n, generator=gen) * 0.02).to(torch.bfloat16)
    oparams = [to_np(p0)]
    oref = oracle.OracleMicroAdam(oparams, m, 1e-3, 64, 0.01, 0, d_block_size=foreign)
    p = torch.nn.Parameter(p0.clone().cuda())
    src = MicroAdam([p], m=m, lr=1e-3, quant_block_size=64)
    src.d_block_size = foreign
    grads = [(torch.randn(n, generator=gen) * 1e-2).to(torch.bfloat16) for _ in range(6)]
    for g in grads[:3]:
        p.grad = g.clone().cuda()
        src.step()
        oref.step([to_np(g)])
    assert src.state[p]["d_block_size"] == foreign
    p2 = torch.nn.Parameter(p.detach().clone())
    dst = MicroAdam([p2], m=m, lr=1e-3, quant_block_size=64)   # d_block_size 20480
    dst.load_state_dict(src.state_dict())
    for s, g in enumerate(grads[3:]):
        p2.grad = g.clone().cuda()
        dst.step()
        assert dst._fusable(p2, dst.state[p2]) == 0
        oref.step([to_np(g)])
        assert_state_equal(dst.state[p2], oref.state[0], f"resumed step {s + 1}")
        assert np.array_equal(to_np(p2.data), oparams[0]), f"resumed step {s + 1}"


def test_cpu_parameter_is_rejected():
    from ista_daslab_optimizers import MicroAdam
    p = torch.nn.Parameter(torch.zeros(100))
    opt = MicroAdam([p], m=3, lr=1e-3, quant_block_size=64)
    p.grad = torch.ones(100)
    with pytest.raises(RuntimeError):
        opt.step()


def test_unaligned_views_take_the_general_route(oracle):
    """Parameters and gradients that are views at an odd element offset (not 16-byte aligned)
    cannot use the vector paths of the fused kernels; the step must still match."""
    from ista_daslab_optimizers import MicroAdam
    gen = torch.Generator().manual_seed(11)
    n, m, q = 5000, 3, 64
    p0 = (torch.randn(n, generator=gen) * 0.02).to(torch.bfloat16)
    oparams = [to_np(p0)]
    oref = oracle.OracleMicroAdam(oparams, m, 1e-3, q, 0.02, 0, d_block_size=2048)
    pbuf = torch.zeros(n + 8, dtype=torch.bfloat16, device="cuda")
    pbuf[3:3 + n] = p0.cuda()
    gp = torch.nn.Parameter(pbuf[3:3 + n])
    assert gp.data_ptr() % 16 != 0
    opt = MicroAdam([gp], m=m, lr=1e-3, quant_block_size=q, k_init=0.02)
    opt.d_block_size = 2048
    for s in range(5):
        g = (torch.randn(n, generator=gen) * 1e-2).to(torch.bfloat16)
        gbuf = torch.zeros(n + 8, dtype=torch.bfloat16, device="cuda")
        gbuf[1:1 + n] = g.cuda()
        gp.grad = gbuf[1:1 + n]
        opt.step()
        oref.step([to_np(g)])
        assert opt._fusable(gp, opt.state[gp]) == 0
        assert_state_equal(opt.state[gp], oref.state[0], f"step {s + 1}")
        assert np.array_equal(to_np(gp.data), oparams[0])


@pytest.mark.parametrize("use_fused", [True, False], ids=["fused", "opbyop"])
def test_window_rows_that_name_the_same_coordinates(oracle, use_fused):
    """Gradients with the same dominant coordinates in every step: every window row names the
    same coordinates, so almost all window entries share their coordinate with other rows
    (the reserve path of the one-pass window stage, where the short list overflows)."""
    from ista_daslab_optimizers import MicroAdam
    gen = torch.Generator().manual_seed(21)
    n, m = 20480 * 2 + 4096, 10
    p0 = (torch.randn(n, generator=gen) * 0.02).to(torch.bfloat16)
    spikes = torch.randperm(n, generator=gen)[: n // 100]
    oparams = [to_np(p0)]
    oref = oracle.OracleMicroAdam(oparams, m, 1e-3, 64, 0.01, 0, d_block_size=20480)
    gp = torch.nn.Parameter(p0.clone().cuda())
    opt = MicroAdam([gp], m=m, lr=1e-3, quant_block_size=64, k_init=0.01)
    opt.use_fused = use_fused
    for s in range(13):
        g = torch.randn(n, generator=gen) * 1e-3
        g[spikes] += torch.sign(torch.randn(spikes.numel(), generator=gen)) * (1.0 + 0.01 * s)
        g = g.to(torch.bfloat16)
        gp.grad = g.clone().cuda()
        opt.step()
        oref.step([to_np(g)])
        assert_state_equal(opt.state[gp], oref.state[0], f"step {s + 1}")
        assert np.array_equal(to_np(gp.data), oparams[0]), f"step {s + 1}"
    # the window really is that repetitive: the rows of a block name nearly the same coordinates
    I = opt.state[gp]["I"][:, :205].long()
    common = sum(len(set(I[0].tolist()) & set(I[r].tolist())) for r in range(1, m)) / (205 * (m - 1))
    assert common > 0.8, common


LOGGING_CASES = [
    # sizes, dtype, m, q, alpha, wd, route
    ([20480 * 2 + 4096, 768, 1001], torch.bfloat16, 4, 64, 0.0, 0.01, "fused"),
    ([20480 + 300], torch.float32, 3, 32, 0.0, 0.0, "fused"),
    ([20480 * 2 + 4096, 768], torch.bfloat16, 4, 64, 0.5, 0.0, "densified"),
    ([5000], torch.float32, 3, 64, 0.25, 0.01, "densified"),
    ([20480 * 3 + 100], torch.bfloat16, 4, 24576, 0.0, 0.01, "spanning"),
    ([20480 * 5 + 77, 4096], torch.bfloat16, 4, 100000, 0.3, 0.0, "spanning"),
    ([20480 * 2 + 4096, 300], torch.bfloat16, 4, 64, -2, 0.01, "quant_err"),
    ([20480 + 77], torch.float32, 3, 32, -2, 0.0, "quant_err"),
    ([20480 * 2 + 8192], torch.bfloat16, 20, 32, 0.0, 0.0, "fused"),   # 5 %: no coordinate cells
    ([20480 * 2 + 3000], torch.bfloat16, 4, 2048, 0.0, 0.01, "fused"),  # long quantisation blocks
]


@pytest.mark.parametrize("use_fused", [True, False], ids=["fused", "opbyop"])
@pytest.mark.parametrize("sizes,dtype,m,q,alpha,wd,route", LOGGING_CASES)
def test_logged_sums_match_oracle(oracle, sizes, dtype, m, q, alpha, wd, route, use_fused):
    """Logging steps (micro_adam.py:155-156, :271-272, :306-308, :320-324, :330-350): the six
    sums handed to _log against the oracle's, which adds the same values in float64.  The
    fused routes form them inside their kernels, in fp32 per block (at most 40 terms per thread,
    then 512 threads pairwise) and in double across blocks: relative error far below the 1e-5
    asked here.  The op-by-op route takes torch's norm of the buffer, whose result has the
    buffer's type (as in the reference): bf16 results, squared and added in bf16, 3e-2.  The zero counts are exact on both, and the step's
    state is the oracle's on logging steps as on any other."""
    from ista_daslab_optimizers import MicroAdam
    k_init = 0.05 if m == 20 else 0.01
    gen = torch.Generator().manual_seed(11)
    cpu_params = [(torch.randn(n, generator=gen) * 0.02).to(dtype) for n in sizes]
    oparams = [to_np(p) for p in cpu_params]
    oref = oracle.OracleMicroAdam(oparams, m, 1e-3, q, k_init, alpha, weight_decay=wd,
                                  d_block_size=20480)
    params = [torch.nn.Parameter(p.clone().cuda()) for p in cpu_params]
    opt = MicroAdam(params, m=m, lr=1e-3, quant_block_size=q, k_init=k_init, alpha=alpha,
                    weight_decay=wd)
    opt.use_fused = use_fused
    opt.log_interval = 2
    opt._logging_active = lambda: True
    logged = []
    opt._log = lambda *a: logged.append([float(x) for x in a[:6]])
    kernel_steps = []
    inner = opt._fused_step
    opt._fused_step = lambda *a, **kw: (kernel_steps.append(opt.steps), inner(*a, **kw))
    wanted = []
    for s in range(6):
        grads = [(torch.randn(n, generator=gen) * 0.01).to(dtype) for n in sizes]
        if s == 3:
            grads[0][: sizes[0] // 2] = 0  # zeros in the gradient: exact zeros may reach u
        for p, g in zip(params, grads):
            p.grad = g.clone().cuda()
        opt.step()
        out = oref.step([to_np(g) for g in grads], metrics=(s + 1) % 2 == 0)
        if out is not None:
            wanted.append(out)
        for i, p in enumerate(params):
            assert_state_equal(opt.state[p], oref.state[i], f"step {s + 1} tensor {i}")
            assert np.array_equal(to_np(p.data), oparams[i]), f"step {s + 1} tensor {i}"
    # every step, logging or not, took the route under test
    assert sorted(set(kernel_steps)) == ([1, 2, 3, 4, 5, 6] if use_fused else [])
    assert len(logged) == 3 == len(wanted)
    rel = 1e-5 if use_fused else (3e-2 if dtype == torch.bfloat16 else 1e-4)
    keys = ("norm_qe", "norm_g", "norm_u", "norm_e", "sparsity_u", "sparsity_qe")
    for got, want in zip(logged, wanted):
        for key, value in zip(keys, got):
            if key.startswith("sparsity"):
                assert value == want[key], (key, value, want[key])
            else:
                assert value == pytest.approx(want[key], rel=rel, abs=0), (key, value, want[key])
        assert want["norm_g"] > 0 and want["norm_u"] > 0 and want["norm_e"] > 0
        assert (want["norm_qe"] > 0) == (alpha == -2)
        if alpha <= 0:
            assert want["sparsity_u"] > 0


@functools.lru_cache(maxsize=None)
def _boundary_gradient(dtype, q):
    """Quantisation blocks of q elements that hold 0, M and the values around the rounding
    boundaries (k + 1/2) M / 15, for M over bf16 significands x all binary exponents."""
    sig = [1.0, 1.0078125, 1.25, 1.5, 1.9921875, 1.328125, 1.7109375]
    if q > 4096:
        sig = [1.0, 1.5, 1.9921875]
    exps = list(range(-126, 127))
    gen = torch.Generator().manual_seed(17)
    per_block = min(15, (q - 6) // 3)       # boundaries one block has room for
    turns = [list(range(i, min(i + per_block, 15))) for i in range(0, 15, per_block)]
    blocks = []
    for e in exps:
        for s_ in sig:
            M = torch.tensor(s_ * 2.0 ** e, dtype=torch.float64).to(dtype)
            u = (M.float() - 0.0) / 15.0
            for ks in turns:
                vals = [torch.zeros((), dtype=dtype)] + [M] * (8 if q >= 64 else 5)
                for k in ks:
                    x = ((k + 0.5) * u.double()).to(dtype)
                    lo = torch.nextafter(x.float(), torch.tensor(0.0)).to(dtype) if dtype == torch.float32 \
                        else (x.view(torch.int16) - 1).view(torch.bfloat16)
                    hi = torch.nextafter(x.float(), torch.tensor(float("inf"))).to(dtype) if dtype == torch.float32 \
                        else (x.view(torch.int16) + 1).view(torch.bfloat16)
                    vals += [lo, x, hi]
                rnd = (torch.rand(q - len(vals), generator=gen).double() * M.double()).to(dtype)
                blk = torch.cat([torch.stack(vals), rnd])
                blocks.append(blk[torch.randperm(q, generator=gen)])
    return torch.cat(blocks)


BOUNDARY_CASES = [
    # DB, q, alpha, use_fused, route the tensor must take (0 op by op, 1 fused, 2 spanning,
    # 3 fused densified)
    (4096, 64, 0.0, True, 1),      # one-chunk kernel, quantisation group size at run time
    (4096, 64, 0.0, False, 0),
    (20480, 64, 0.0, True, 1),     # hardware block, group of 8 lanes compiled in, statistics
    (20480, 32, 0.0, True, 1),     # shared across lanes; group of 4 lanes
    (20480, 2048, 0.0, True, 1),   # quantisation blocks longer than a wave's stretch
    (20480, 1024, 0.0, True, 1),
    (20480, 64, 0.5, True, 3),     # both quantisations of the densified step
    (20480, 2048, 0.5, True, 3),
    (20480, 24576, 0.0, True, 2),  # two-pass route: statistics across top-k blocks
    (20480, 24576, 0.5, True, 2),  # ... and the 2 x 16 table of its second pass
]


@pytest.mark.parametrize("DB,q,alpha,use_fused,route", BOUNDARY_CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_quantisation_rounding_boundaries(oracle, dtype, DB, q, alpha, use_fused, route):
    """The 4-bit codes where they are hardest to get right: every quantisation block holds its
    minimum 0, its maximum M, and for the 15 rounding boundaries the value nearest to
    (k + 1/2) u and its two neighbours (u = (M - 0) / 15 as the kernels form it; blocks too short
    for all 15 take them in turns), with M running through bf16 significands and through every
    binary exponent from -126 to 126, so that steps u that are subnormal, tiny, ordinary and huge
    all occur.  The fused kernels divide by a shared reciprocal where the oracle divides; the
    codes must agree bit for bit all the same, in every kernel instance that forms statistics or
    codes in its own way.  A second step with a zero gradient dequantises and requantises them."""
    from ista_daslab_optimizers import MicroAdam
    g0 = _boundary_gradient(dtype, q)
    pad = (-g0.numel()) % DB
    if q <= DB:  # whole top-k blocks, so that the full-block kernel instances run
        g0 = torch.cat([g0, torch.zeros(pad, dtype=dtype)])
    assert torch.isfinite(g0.float()).all()
    d = g0.numel()
    p0 = (torch.randn(d, generator=torch.Generator().manual_seed(18)) * 0.02).to(dtype)
    oparams = [to_np(p0)]
    oref = oracle.OracleMicroAdam(oparams, 4, 1e-3, q, 0.001, alpha, d_block_size=DB)
    gp = torch.nn.Parameter(p0.clone().cuda())
    opt = MicroAdam([gp], m=4, lr=1e-3, quant_block_size=q, k_init=0.001, alpha=alpha)
    opt.d_block_size = DB
    opt.use_fused = use_fused
    for step, g in enumerate([g0, torch.zeros_like(g0), g0]):
        gp.grad = g.clone().cuda()
        opt.step()
        assert (opt._fusable(gp, opt.state[gp]) if use_fused else 0) == route
        oref.step([to_np(g)])
        assert_state_equal(opt.state[gp], oref.state[0], f"step {step + 1}")
        assert np.array_equal(to_np(gp.data), oparams[0]), f"step {step + 1}: parameters"
    codes = oracle.unpack_codes(to_np(opt.state[gp]["error"]), d)
    assert set(np.unique(codes)) == set(range(16))
