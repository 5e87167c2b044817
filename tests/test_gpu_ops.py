"""GPU parity, one entry point of the C ABI at a time, against the CPU oracle.

Everything here is bit-exact: integer indices, 4-bit codes, bf16 bit patterns and fp32 words
must equal the oracle's on the same seeded inputs.  Calls go through the package's ctypes
binding of libmicroadam_hip.so (and the extension-module stand-ins built on it).
"""
import numpy as np
import pytest
import torch

from gpu_util import to_np, to_torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def hip():
    from ista_daslab_optimizers import _hip
    return _hip


@pytest.fixture(scope="module")
def ext():
    import ista_daslab_cuda_micro_adam
    import ista_daslab_cuda_tools
    return ista_daslab_cuda_tools, ista_daslab_cuda_micro_adam


def _vec(seed, n, dtype, scale=1e-2):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, generator=g) * scale).to(dtype)


def test_device_queries(ext):
    tools, _ = ext
    assert tools.get_sm_count() == torch.cuda.get_device_properties(0).multi_processor_count
    assert tools.get_max_floats_for_shared_memory_per_thread_block() == 40960


def test_bf16_rounding_on_device(hip, oracle):
    """The device's fp32 -> bf16 narrowing (copy_values d2k on fp32 input) is RNE like the
    oracle's, including halfway cases and denormal-range values."""
    import ista_daslab_cuda_tools as tools
    g = torch.Generator().manual_seed(7)
    x = torch.randn(1 << 16, generator=g) * torch.logspace(-20, 20, 1 << 16)
    x[:6] = torch.tensor([1.00390625, 1.01171875, -1.00390625, 0.0, 3.0e38, 1e-39])
    xd = x.cuda()
    n = x.numel()
    idx = torch.arange(n, dtype=torch.int32).remainder(32768).to(torch.int16).cuda()
    out = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
    tools.copy_values(n, n, 32768, 32768, idx, xd, out, 1)
    assert np.array_equal(to_np(out), oracle.f32_to_bf16(x.numpy()))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d,q", [(4096, 64), (1000, 64), (1001, 32), (40, 64), (99999, 1000),
                                 (20480 * 3 + 100, 100000), (7, 3)])
def test_quant_minmax_quantinv(ext, hip, oracle, dtype, d, q):
    _, ma = ext
    x = _vec(d + q, d, dtype)
    xo = to_np(x)
    xd = x.cuda()
    nb = (d + q - 1) // q
    mn = torch.zeros(nb + 1, dtype=torch.bfloat16, device="cuda")
    mx = torch.zeros(nb + 1, dtype=torch.bfloat16, device="cuda")
    omn, omx = np.zeros(nb + 1, np.uint16), np.zeros(nb + 1, np.uint16)
    hip.check(hip.lib.ma_block_minmax(d, q, hip.dev_ptr(xd), hip.dev_ptr(mn), hip.dev_ptr(mx),
                                      hip.dtype_tag(xd), hip.stream_ptr()), "minmax")
    oracle.block_minmax(d, q, xo, omn, omx)
    assert np.array_equal(to_np(mn), omn) and np.array_equal(to_np(mx), omx)

    xq = torch.zeros((d + 1) // 2, dtype=torch.uint8, device="cuda")
    oxq = np.zeros((d + 1) // 2, np.uint8)
    ma.asymm_block_quant(d, q, xq, mn, mx, xd)
    oracle.asymm_block_quant(d, q, oxq, omn, omx, xo)
    assert np.array_equal(to_np(xq), oxq)

    for alpha in (1.0, 0.5, 0.3):
        acc = _vec(d + 1, d, dtype)
        oacc = to_np(acc)
        accd = acc.cuda()
        ma.asymm_block_quant_inv(d, q, xq, mn, mx, accd, alpha)
        oracle.asymm_block_quant_inv(d, q, oxq, omn, omx, oacc, alpha)
        assert np.array_equal(to_np(accd), oacc), alpha


@pytest.mark.parametrize("dtype", DTYPES)
def test_quant_unaligned_view(ext, oracle, dtype):
    """Views that start off the 16-byte grid take the element-wise load path."""
    _, ma = ext
    d, q = 3001, 64
    buf = _vec(3, d + 3, dtype).cuda()
    x = buf[3:]
    xo = to_np(x)
    nb = (d + q - 1) // q
    mn = (_vec(4, nb + 1, torch.bfloat16) - 0.02).cuda()
    mx = mn + 0.04
    xq = torch.zeros((d + 1) // 2, dtype=torch.uint8, device="cuda")
    oxq = np.zeros((d + 1) // 2, np.uint8)
    ma.asymm_block_quant(d, q, xq, mn, mx, x)
    oracle.asymm_block_quant(d, q, oxq, to_np(mn), to_np(mx), xo)
    assert np.array_equal(to_np(xq), oxq)
    ma.asymm_block_quant_inv(d, q, xq, mn, mx, x, 1.0)
    oracle.asymm_block_quant_inv(d, q, oxq, to_np(mn), to_np(mx), xo, 1.0)
    assert np.array_equal(to_np(x), xo)
    assert np.array_equal(to_np(buf[:3]), to_np(_vec(3, d + 3, dtype)[:3]))


TOPK_CASES = [
    # d, DB, k_init
    (5000, 1024, 0.03),
    (20480 * 2 + 4096, 20480, 0.01),
    (768, 20480, 0.01),
    (32768 + 5, 32768, 0.01),
    (3 * 4096 + 1, 4096, 0.05),
    (10240 * 2 + 77, 10240, 0.01),
    (2000, 512, 1.0),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d,DB,k_init", TOPK_CASES)
@pytest.mark.parametrize("kind", ["normal", "ties", "zeros", "sparse"])
def test_block_topk_gather_zero(hip, oracle, dtype, d, DB, k_init, kind):
    x = _vec(d, d, dtype, 1e-3)
    if kind == "ties":
        x = (torch.round(x.float() * 4000) / 4000).to(dtype)
    elif kind == "zeros":
        x.zero_()
    elif kind == "sparse":
        g = torch.Generator().manual_seed(1)
        x[torch.rand(d, generator=g) < 0.995] = 0
    geo = oracle.geometry(d, DB, k_init, 64)
    dbs, km, kf, k = geo["d_block_size"], geo["k_block_size_many"], geo["k_block_size_few"], geo["k"]
    xo = to_np(x)
    oI = np.zeros(k, np.int16)
    oV = np.zeros(k, np.uint16)
    oracle.block_topk(d, dbs, km, kf, xo, oI)
    oracle.copy_values(d, k, dbs, km, oI, xo, oV, 1)
    oracle.zerorize_block_components(xo, oI, d, k, dbs, km)

    xd = x.cuda()
    I = torch.full((k,), -1, dtype=torch.int16, device="cuda")
    V = torch.zeros(k, dtype=torch.bfloat16, device="cuda")
    hip.check(hip.lib.ma_block_topk(d, dbs, km, kf, hip.dev_ptr(xd), hip.dev_ptr(I), hip.dev_ptr(V),
                                    1, hip.dtype_tag(xd), hip.stream_ptr()), "topk")
    assert np.array_equal(to_np(I), oI)
    assert np.array_equal(to_np(V), oV)
    assert np.array_equal(to_np(xd), xo)

    # indices only: x untouched
    xd2 = x.cuda()
    I2 = torch.zeros(k, dtype=torch.int16, device="cuda")
    hip.check(hip.lib.ma_block_topk(d, dbs, km, kf, hip.dev_ptr(xd2), hip.dev_ptr(I2), None, 0,
                                    hip.dtype_tag(xd2), hip.stream_ptr()), "topk")
    assert np.array_equal(to_np(I2), oI) and np.array_equal(to_np(xd2), to_np(x))


@pytest.mark.parametrize("dtype", DTYPES)
def test_copy_values_and_zerorize(ext, oracle, dtype):
    tools, _ = ext
    rng = np.random.default_rng(2)
    d, DB, km, kf = 2500, 1000, 7, 4
    k = 2 * km + kf
    idx = np.concatenate([rng.choice(1000, km, replace=False), rng.choice(1000, km, replace=False),
                          rng.choice(500, kf, replace=False)]).astype(np.int16)
    x = _vec(5, d, dtype)
    xo = to_np(x)
    xd, idxd = x.cuda(), torch.from_numpy(idx).cuda()
    out = torch.zeros(k, dtype=torch.bfloat16, device="cuda")
    oout = np.zeros(k, np.uint16)
    tools.copy_values(d, k, DB, km, idxd, xd, out, 1)
    oracle.copy_values(d, k, DB, km, idx, xo, oout, 1)
    assert np.array_equal(to_np(out), oout)
    back = torch.zeros(d, dtype=dtype, device="cuda")
    oback = np.zeros_like(xo)
    tools.copy_values(d, k, DB, km, idxd, out, back, 0)
    oracle.copy_values(d, k, DB, km, idx, oout, oback, 0)
    assert np.array_equal(to_np(back), oback)
    tools.zerorize_block_components(xd, idxd, d, k, DB, km)
    oracle.zerorize_block_components(xo, idx, d, k, DB, km)
    assert np.array_equal(to_np(xd), xo)


def _window(rng, m, nblocks, dbs, kb, tail, kfew):
    k = nblocks * kb + kfew
    I = np.zeros((m, k), dtype=np.int16)
    for r in range(m):
        for b in range(nblocks):
            I[r, b * kb:(b + 1) * kb] = rng.choice(dbs, kb, replace=False)
        if kfew:
            I[r, nblocks * kb:] = rng.choice(tail, kfew, replace=False)
    return I, k


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,dbs,kb,nblocks,tail,kfew,t", [
    (10, 300, 12, 3, 100, 5, 1), (10, 300, 12, 3, 100, 5, 7), (10, 300, 12, 3, 100, 5, 10),
    (10, 300, 12, 3, 100, 5, 23), (10, 20480, 205, 2, 4096, 41, 15),
    (20, 20480, 1024, 2, 0, 0, 40),      # m * kb > 4096: the block is walked in coordinate ranges
    (4, 32768, 3000, 1, 100, 10, 9), (3, 64, 64, 2, 0, 0, 5),
])
def test_compute_microadam_update(ext, oracle, dtype, m, dbs, kb, nblocks, tail, kfew, t):
    _, ma = ext
    rng = np.random.default_rng(t + m)
    d = nblocks * dbs + tail
    I, k = _window(rng, m, nblocks, dbs, kb, tail, kfew)
    V = oracle.f32_to_bf16((rng.standard_normal(m * k) * 1e-2).astype(np.float32)).reshape(m, k)
    out = torch.full((d,), 3.0, dtype=dtype, device="cuda")  # untouched cells must keep this
    oout = to_np(torch.full((d,), 3.0, dtype=dtype))
    ma.compute_microadam_update(1, 512, 100, t, 0.9, 0.999, 1e-8, dbs, kb, d, m, k,
                                torch.from_numpy(I).cuda(), to_torch(V.reshape(-1)).view(m, k), out)
    oracle.compute_microadam_update(t, 0.9, 0.999, 1e-8, dbs, kb, d, m, k, I, V, oout)
    assert np.array_equal(to_np(out), oout)


@pytest.mark.parametrize("eps", [1e-8, 0.0, 1e-30, 1.0])
@pytest.mark.parametrize("dtype", DTYPES)
def test_adam_direction_over_many_magnitudes(ext, oracle, dtype, eps):
    """The direction (z1 s1) / (eps + sqrt(z2 s2)) of compute_microadam_update
    (micro_adam.py:277-291) on 4 million coordinates whose window values run over 30 decades, down
    to values whose squares are subnormal or vanish, every coordinate named by all three rows (so
    the sums cancel to all sizes).  For bf16 updates the kernels settle the rounding from an
    approximate quotient and take the exactly rounded way only near a tie: the bits must be the
    oracle's (correctly rounded square root and division) everywhere all the same."""
    _, ma = ext
    rng = np.random.default_rng(123)
    m, dbs, nblocks, t = 3, 4096, 1024, 7
    d = k = nblocks * dbs
    I = np.stack([np.tile(rng.permutation(dbs).astype(np.int16), nblocks) for _ in range(m)])
    mag = 10.0 ** rng.uniform(-24, 6, size=(m, k))
    mag[:, : k // 8] = 10.0 ** rng.uniform(-3, -1, size=(m, k // 8))   # ordinary gradients
    val = (mag * rng.choice([-1.0, 1.0], size=(m, k))).astype(np.float32)
    val[0, k // 8: k // 4] = -val[1, k // 8: k // 4]                    # sums that nearly cancel
    V = oracle.f32_to_bf16(val.reshape(-1)).reshape(m, k)
    out = torch.zeros(d, dtype=dtype, device="cuda")
    oout = to_np(torch.zeros(d, dtype=dtype))
    ma.compute_microadam_update(1, 512, 100, t, 0.9, 0.999, eps, dbs, dbs, d, m, k,
                                torch.from_numpy(I).cuda(), to_torch(V.reshape(-1)).view(m, k), out)
    oracle.compute_microadam_update(t, 0.9, 0.999, eps, dbs, dbs, d, m, k, I, V, oout)
    got = to_np(out)
    bad = np.nonzero(got != oout)[0]
    assert bad.size == 0, (bad.size, bad[:5], got[bad[:5]], oout[bad[:5]])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d", [8192, 1001, 5])
def test_param_update(hip, oracle, dtype, d):
    p, u = _vec(1, d, dtype, 0.02), _vec(2, d, dtype, 1.0)
    u[::3] = 0
    lr, wd = 1e-3, 0.1
    for decay in (0, 1):
        po = to_np(p)
        pd, ud = p.cuda(), u.cuda()
        hip.check(hip.lib.ma_param_update(d, hip.dev_ptr(pd), hip.dev_ptr(ud), -lr, decay,
                                          1 - lr * wd, hip.dtype_tag(pd), hip.stream_ptr()), "upd")
        if decay:
            oracle.weight_decay(po, np.float32(1 - lr * wd))
        oracle.param_update(po, to_np(u), np.float32(-lr))
        assert np.array_equal(to_np(pd), po)


def test_argument_errors(hip, ext):
    tools, ma = ext
    x = torch.zeros(100, device="cuda")
    with pytest.raises(RuntimeError):
        ma.asymm_block_quant_inv(100, 64, torch.zeros(50, dtype=torch.uint8), torch.zeros(3, dtype=torch.bfloat16),
                                 torch.zeros(3, dtype=torch.bfloat16), torch.zeros(100), 1.0)  # CPU tensors
    with pytest.raises(TypeError):
        ma.asymm_block_quant_inv(100, 64, torch.zeros(50, dtype=torch.uint8, device="cuda"),
                                 torch.zeros(3, device="cuda"), torch.zeros(3, device="cuda"), x, 1.0)
    assert hip.lib.ma_block_topk(100, 40000, 1, 0, hip.dev_ptr(x), hip.dev_ptr(x), None, 0, 0, None) != 0
    assert hip.lib.ma_compute_microadam_update(1, 1, 1, 1, 0.9, 0.999, 1e-8, 64, 4, 100, 65, 8,
                                               hip.dev_ptr(x), hip.dev_ptr(x), hip.dev_ptr(x), 0, None) == -3
    assert "window" in hip.error_string(-3)
