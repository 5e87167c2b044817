"""Pins for the CPU oracle (oracle/microadam_oracle.c).

The reference holds no tests or golden vectors for MicroAdam, and its device arithmetic
sits in an un-vendored CUDA package, so each oracle function is pinned here by what the
mathematics fixes: closed forms, invariants, brute force on small inputs, library
routines (numpy / torch CPU) and a second op-for-op statement in torch
(tests/torch_restatement.py).  Each check is chosen so that a plausible slip (dropped
+0.5, /16 for /15, swapped nibbles, wrong age, transposed window) fails it.
"""
import math

import numpy as np
import pytest
import torch

from torch_restatement import TorchMicroAdam


def bits(t):
    """torch bf16/fp32 CPU tensor -> numpy array the oracle takes."""
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()
    return t.contiguous().numpy().copy()


def from_bits(a):
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    return torch.from_numpy(a.copy())


# ---- rounding helpers ---------------------------------------------------------

def test_bf16_rounding_matches_torch(oracle):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(200000, generator=g) * torch.logspace(-30, 30, 200000)
    x[:8] = torch.tensor([0.0, -0.0, 1.0, 1.00390625, 1.01171875, float("inf"), -float("inf"),
                          3.3895313892515355e38])
    want = bits(x.to(torch.bfloat16))
    got = oracle.f32_to_bf16(x.numpy())
    assert np.array_equal(want, got)
    one = [oracle.lib().ora_f32_to_bf16(float(v)) for v in x[:64]]
    assert one == list(want[:64])
    assert np.array_equal(oracle.bf16_to_f32(want), x.to(torch.bfloat16).float().numpy())


# ---- geometry --------------------------------------------------------------------

def test_block_split_quirks(oracle):
    # tools.py:85-92
    assert oracle.block_split(5, 10) == (1, 5)
    assert oracle.block_split(10, 10) == (1, 10)
    assert oracle.block_split(25, 10) == (2, 20)
    assert oracle.block_split(16777216, 20480) == (819, 16773120)


@pytest.mark.parametrize("d,DB,k_init,q,want", [
    # closed-form rows worked by hand from micro_adam.py:77-94
    (16777216, 20480, 0.01, 64, dict(d_block_size=20480, topk_full_blocks_count=819,
                                     d_index_topk=16773120, k_block_size_many=205,
                                     k_block_size_few=41, k_index=167895, k=167936,
                                     quant_full_blocks_count=262144, d_index_quant=16777216,
                                     error_bytes=8388608, stats_len=262145)),
    (1048576, 20480, 0.01, 64, dict(topk_full_blocks_count=51, d_index_topk=1044480,
                                    k_block_size_few=41, k=10496)),
    (768, 20480, 0.01, 64, dict(d_block_size=768, topk_full_blocks_count=1, d_index_topk=768,
                                k_block_size_many=8, k_block_size_few=0, k=8,
                                quant_full_blocks_count=12, d_index_quant=768, stats_len=13)),
    (4096, 20480, 0.01, 100000, dict(d_block_size=4096, k=41, quant_full_blocks_count=1,
                                     d_index_quant=4096, stats_len=2)),
    (16777216, 20480, 0.01, 100000, dict(quant_full_blocks_count=167, d_index_quant=16700000,
                                         stats_len=168)),
    (2048 * 8192, 20480, 0.05, 32, dict(k_block_size_many=1024, topk_full_blocks_count=819,
                                        k_block_size_few=205, k=819 * 1024 + 205)),
    (7, 20480, 0.01, 64, dict(d_block_size=7, k_block_size_many=1, k=1, error_bytes=4,
                              quant_full_blocks_count=1, d_index_quant=7)),
])
def test_geometry_closed_forms(oracle, d, DB, k_init, q, want):
    g = oracle.geometry(d, DB, k_init, q)
    for key, val in want.items():
        assert g[key] == val, key


def test_geometry_invariants(oracle):
    rng = np.random.default_rng(0)
    for _ in range(300):
        d = int(rng.integers(1, 200000))
        DB = int(rng.integers(1, 32769))
        q = int(rng.integers(1, 5000))
        k_init = float(rng.choice([0.01, 0.05, 0.3, 1.0]))
        g = oracle.geometry(d, DB, k_init, q)
        dbs = g["d_block_size"]
        assert dbs == min(d, DB)
        assert g["k_block_size_few"] <= g["k_block_size_many"] <= dbs
        assert g["k_index"] + g["k_block_size_few"] == g["k"]
        assert g["topk_full_blocks_count"] * dbs + (d - g["d_index_topk"]) == d
        assert 0 <= d - g["d_index_topk"] < dbs
        assert g["error_bytes"] == (d + 1) // 2


# ---- top-k ----------------------------------------------------------------------

def brute_topk(xf, n_full, dbs, k_many, k_few):
    """Stable descending sort on |x| per block: ties keep the lowest index."""
    out = []
    d = xf.size
    for b in range(n_full + (1 if k_few > 0 else 0)):
        blk = np.abs(xf[b * dbs:min((b + 1) * dbs, d)])
        kb = k_many if b < n_full else k_few
        order = np.argsort(-blk.astype(np.float64), kind="stable")[:kb]
        out.append(np.sort(order))
    return np.concatenate(out).astype(np.int16)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("case", ["normal", "ties", "zeros", "const", "kfull", "sparse"])
def test_block_topk_against_stable_sort(oracle, dtype, case):
    rng = np.random.default_rng(hash((dtype, case)) % 2**32)
    d, DB, k_init = 5000, 1024, 0.03
    if case == "kfull":
        k_init = 1.0
    x = rng.standard_normal(d).astype(np.float32)
    if case == "ties":
        x = np.round(x * 4) / 4
    elif case == "zeros":
        x[:] = 0
    elif case == "const":
        x[:] = -1.5
    elif case == "sparse":
        x[rng.random(d) < 0.995] = 0
    arr = oracle.f32_to_bf16(x) if dtype == "bf16" else x
    xf = oracle.bf16_to_f32(arr) if dtype == "bf16" else x
    g = oracle.geometry(d, DB, k_init, 64)
    I = np.full(g["k"], -1, dtype=np.int16)
    oracle.block_topk(d, g["d_block_size"], g["k_block_size_many"], g["k_block_size_few"], arr, I)
    want = brute_topk(xf, g["topk_full_blocks_count"], g["d_block_size"], g["k_block_size_many"],
                      g["k_block_size_few"])
    assert np.array_equal(I, want)


def test_block_topk_bf16_full_block_ties(oracle):
    # a 20480-wide bf16 block has many exact ties at the threshold
    rng = np.random.default_rng(5)
    x = oracle.f32_to_bf16((rng.standard_normal(3 * 20480 + 4096) * 1e-3).astype(np.float32))
    g = oracle.geometry(x.size, 20480, 0.01, 64)
    I = np.zeros(g["k"], dtype=np.int16)
    oracle.block_topk(x.size, 20480, 205, 41, x, I)
    want = brute_topk(oracle.bf16_to_f32(x), 3, 20480, 205, 41)
    assert np.array_equal(I, want)
    # the threshold magnitude really is tied, so the tie rule is exercised
    blk = np.abs(oracle.bf16_to_f32(x[:20480]))
    thr = blk[I[:205]].min()
    assert (blk == thr).sum() > (blk[I[:205]] == thr).sum()


# ---- gather / zero -----------------------------------------------------------------

def test_copy_values_and_zerorize(oracle):
    rng = np.random.default_rng(2)
    d, DB, k_many, k_few = 2500, 1000, 7, 4
    k = 2 * k_many + k_few
    for arr in (rng.standard_normal(d).astype(np.float32),
                oracle.f32_to_bf16(rng.standard_normal(d).astype(np.float32))):
        idx = np.concatenate([rng.choice(1000, k_many, replace=False),
                              rng.choice(1000, k_many, replace=False),
                              rng.choice(500, k_few, replace=False)]).astype(np.int16)
        glob = (np.arange(k) // k_many) * DB + idx
        out = np.zeros(k, dtype=np.uint16)
        oracle.copy_values(d, k, DB, k_many, idx, arr, out, 1)
        t = from_bits(arr)
        assert np.array_equal(out, bits(t[torch.from_numpy(glob)].to(torch.bfloat16)))
        # k2d scatters the bf16 values back
        back = np.zeros_like(arr)
        oracle.copy_values(d, k, DB, k_many, idx, out, back, 0)
        wantb = torch.zeros_like(t)
        wantb[torch.from_numpy(glob)] = from_bits(out).to(t.dtype)
        assert np.array_equal(back, bits(wantb))
        z = arr.copy()
        oracle.zerorize_block_components(z, idx, d, k, DB, k_many)
        want = arr.copy()
        want[glob] = 0
        assert np.array_equal(z, want)


# ---- min / max -----------------------------------------------------------------------

@pytest.mark.parametrize("d,q", [(4096, 64), (1000, 64), (50, 64), (64, 64), (777, 100)])
def test_block_minmax_against_torch(oracle, d, q):
    rng = np.random.default_rng(d + q)
    for arr in (rng.standard_normal(d).astype(np.float32),
                oracle.f32_to_bf16(rng.standard_normal(d).astype(np.float32))):
        t = from_bits(arr)
        nfull, start = (1, d) if d < q else (d // q, d - d % q)
        mn = torch.zeros(nfull + 1, dtype=torch.bfloat16)
        mx = torch.zeros(nfull + 1, dtype=torch.bfloat16)
        # micro_adam.py:217-228, stock torch
        if nfull == 1:
            mn[:1] = t[:start].min()
            mx[:1] = t[:start].max()
        else:
            mn[:nfull] = t[:start].view(nfull, q).min(dim=1).values
            mx[:nfull] = t[:start].view(nfull, q).max(dim=1).values
        if start < d:
            mn[nfull] = t[start:].min()
            mx[nfull] = t[start:].max()
        omn = np.zeros(nfull + 1, dtype=np.uint16)
        omx = np.zeros(nfull + 1, dtype=np.uint16)
        oracle.block_minmax(d, q, arr, omn, omx)
        assert np.array_equal(omn, bits(mn)) and np.array_equal(omx, bits(mx))


# ---- Q / Qinv --------------------------------------------------------------------------

def test_quant_known_answers(oracle):
    q = 16
    # ramp 0..15 with min 0, max 15 (u = 1): code i for element i; nibble order from
    # utils/quantizers.py:24-27 puts element 2j in the high nibble
    x = np.arange(16, dtype=np.float32)
    mn, mx = oracle.f32_to_bf16(np.float32([0])), oracle.f32_to_bf16(np.float32([15]))
    xq = np.zeros(8, dtype=np.uint8)
    oracle.asymm_block_quant(16, q, xq, mn, mx, x)
    assert list(xq) == [0x01, 0x23, 0x45, 0x67, 0x89, 0xAB, 0xCD, 0xEF]
    # round half up: i + 0.4 -> i, i + 0.5 -> i + 1, i + 0.6 -> i + 1
    for frac, bump in ((0.375, 0), (0.5, 1), (0.625, 1)):
        xs = np.minimum(np.arange(16, dtype=np.float32) + np.float32(frac), np.float32(15))
        oracle.asymm_block_quant(16, q, xq, mn, mx, xs)
        assert list(oracle.unpack_codes(xq, 16)) == [min(i + bump, 15) for i in range(16)]
    # divisor is 15: range 30 -> step 2
    mx2 = oracle.f32_to_bf16(np.float32([30]))
    oracle.asymm_block_quant(16, q, xq, mn, mx2, np.arange(16, dtype=np.float32) * 2)
    assert list(oracle.unpack_codes(xq, 16)) == list(range(16))
    # clamp outside the stats, zero range -> code 0
    oracle.asymm_block_quant(4, q, xq, mn, mx, np.float32([-3, 99, 7.2, 0]))
    assert list(oracle.unpack_codes(xq, 4)) == [0, 15, 7, 0]
    oracle.asymm_block_quant(4, q, xq, mx, mx, np.float32([15, 15, 20, -1]))
    assert list(oracle.unpack_codes(xq, 4)) == [0, 0, 0, 0]
    # odd d: the last low nibble is 0
    oracle.asymm_block_quant(3, q, xq, mn, mx, np.float32([1, 2, 3]))
    assert list(xq[:2]) == [0x12, 0x30]
    # Qinv known answers: x += alpha * (code * u + min), min = -1, max = 2 (u = 0.2)
    mn3, mx3 = oracle.f32_to_bf16(np.float32([-1])), oracle.f32_to_bf16(np.float32([2]))
    xq3 = np.array([0x0F, 0x5A], dtype=np.uint8)
    acc = np.float32([10, 10, 10, 10])
    oracle.asymm_block_quant_inv(4, q, xq3, mn3, mx3, acc, 0.5)
    u = np.float32(3) / np.float32(15)
    want = np.float32(10) + np.float32(0.5) * (np.float32([0, 15, 5, 10]) * u + np.float32(-1))
    assert np.array_equal(acc, want.astype(np.float32))
    assert np.allclose(acc, [9.5, 11.0, 10.0, 10.5], atol=1e-6)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("d,q", [(4096, 64), (1000, 64), (1001, 32), (40, 64), (9999, 1000)])
def test_quant_roundtrip_invariants(oracle, dtype, d, q):
    rng = np.random.default_rng(d * 7 + q)
    xf = (rng.standard_normal(d) * 1e-2).astype(np.float32)
    arr = oracle.f32_to_bf16(xf) if dtype == "bf16" else xf
    xf = oracle.bf16_to_f32(arr) if dtype == "bf16" else xf
    nb = (d + q - 1) // q
    mn = np.zeros(nb + 1, dtype=np.uint16)
    mx = np.zeros(nb + 1, dtype=np.uint16)
    oracle.block_minmax(d, q, arr, mn, mx)
    xq = np.zeros((d + 1) // 2, dtype=np.uint8)
    oracle.asymm_block_quant(d, q, xq, mn, mx, arr)
    codes = oracle.unpack_codes(xq, d).astype(np.int64)
    b = np.arange(d) // q
    mnf, mxf = oracle.bf16_to_f32(mn)[b].astype(np.float64), oracle.bf16_to_f32(mx)[b].astype(np.float64)
    u = (mxf - mnf) / 15
    # against a float64 evaluation: the code is the nearest level, except where fp32 rounding
    # may flip an exact half-way case
    ideal = np.clip(np.floor((xf.astype(np.float64) - mnf) / np.where(u == 0, 1, u) + 0.5), 0, 15)
    frac = (xf.astype(np.float64) - mnf) / np.where(u == 0, 1, u) + 0.5
    near_half = np.abs(frac - np.round(frac)) < 1e-4
    assert np.all((codes == ideal) | near_half | (u == 0))
    assert np.all(np.abs(codes - ideal) <= 1)
    if dtype == "bf16":  # stats are exact for bf16 data: extremes map to the end codes
        for blk in range(nb):
            sl = slice(blk * q, min((blk + 1) * q, d))
            if u[sl][0] > 0:
                assert codes[sl][np.argmin(xf[sl])] == 0 and codes[sl][np.argmax(xf[sl])] == 15
    # monotone within a block
    for blk in range(min(nb, 20)):
        sl = slice(blk * q, min((blk + 1) * q, d))
        o = np.argsort(xf[sl], kind="stable")
        assert np.all(np.diff(codes[sl][o]) >= 0)
    # |Qinv(Q(x)) - x| <= u/2 (+ rounding of the stats for fp32 data, + output rounding)
    acc = np.zeros_like(arr)
    oracle.asymm_block_quant_inv(d, q, xq, mn, mx, acc, 1.0)
    deq = oracle.bf16_to_f32(acc) if dtype == "bf16" else acc
    inside = (xf >= mnf) & (xf <= mxf)
    tol = u / 2 + np.abs(xf) * (2.0 ** -8 if dtype == "bf16" else 2.0 ** -22) + 1e-12
    assert np.all(np.abs(deq.astype(np.float64) - xf)[inside] <= tol[inside] * 1.001)


# ---- Adam direction -----------------------------------------------------------------------

def _window(rng, m, nblocks, dbs, kb, tail, kfew):
    """Random valid window: distinct indices per row and block."""
    k = nblocks * kb + kfew
    I = np.zeros((m, k), dtype=np.int16)
    for r in range(m):
        for b in range(nblocks):
            I[r, b * kb:(b + 1) * kb] = rng.choice(dbs, kb, replace=False)
        if kfew:
            I[r, nblocks * kb:] = rng.choice(tail, kfew, replace=False)
    return I, k


@pytest.mark.parametrize("t", [1, 3, 10, 11, 25])
def test_adam_direction_against_float64_window_sum(oracle, t):
    rng = np.random.default_rng(t)
    m, dbs, kb, nblocks, tail, kfew = 10, 300, 12, 3, 100, 5
    d = nblocks * dbs + tail
    I, k = _window(rng, m, nblocks, dbs, kb, tail, kfew)
    Vf = (rng.standard_normal((m, k)) * 1e-2).astype(np.float32)
    V = oracle.f32_to_bf16(Vf.reshape(-1)).reshape(m, k)
    Vf = oracle.bf16_to_f32(V.reshape(-1)).reshape(m, k).astype(np.float64)
    b1, b2, eps = 0.9, 0.999, 1e-8
    out = np.zeros(d, dtype=np.float32)
    oracle.compute_microadam_update(t, b1, b2, eps, dbs, kb, d, m, k, I, V, out)
    z1 = np.zeros(d)
    z2 = np.zeros(d)
    hit = np.zeros(d, dtype=bool)
    base = (np.arange(k) // kb) * dbs
    for r in range(min(t, m)):
        age = (t - 1 - r) % m
        pos = base + I[r]
        z1[pos] += b1 ** age * Vf[r]
        z2[pos] += b2 ** age * Vf[r] ** 2
        hit[pos] = True
    want = ((1 - b1) * z1 / (1 - b1 ** t)) / (eps + np.sqrt((1 - b2) * z2 / (1 - b2 ** t)))
    assert np.all(out[~hit] == 0)
    # fp32 sums of up to m terms, with cancellation in z1: absolute slack on O(1) outputs
    assert np.allclose(out[hit], want[hit], rtol=5e-6, atol=2e-6)
    # rows beyond min(t, m) are ignored: scribbling on them changes nothing
    if t < m:
        I2, V2 = I.copy(), V.copy()
        V2[t:] = 0x4000
        out2 = np.zeros(d, dtype=np.float32)
        oracle.compute_microadam_update(t, b1, b2, eps, dbs, kb, d, m, k, I2, V2, out2)
        assert np.array_equal(out, out2)
    # the order of entries inside a block row does not matter
    perm = rng.permutation(kb)
    I3, V3 = I.copy(), V.copy()
    I3[:, :kb], V3[:, :kb] = I[:, :kb][:, perm], V[:, :kb][:, perm]
    out3 = np.zeros(d, dtype=np.float32)
    oracle.compute_microadam_update(t, b1, b2, eps, dbs, kb, d, m, k, I3, V3, out3)
    assert np.array_equal(out, out3)


def test_dense_limit_is_adam(oracle):
    """k_init = 1: every coordinate is kept, EF stays empty, and for t <= m the update
    is dense Adam's (torch.optim.Adam on the same bf16-representable gradients)."""
    rng = np.random.default_rng(11)
    d, m, lr = 1500, 6, 1e-2
    p0 = (rng.standard_normal(d) * 0.1).astype(np.float32)
    p = p0.copy()
    opt = oracle.OracleMicroAdam([p], m=m, lr=lr, quant_block_size=64, k_init=1.0, d_block_size=512)
    tp = torch.nn.Parameter(torch.from_numpy(p0.copy()))
    adam = torch.optim.Adam([tp], lr=lr, betas=(0.9, 0.999), eps=1e-8)
    for t in range(1, m + 1):
        g = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.standard_normal(d).astype(np.float32)))
        tp.grad = torch.from_numpy(g.copy())
        adam.step()
        opt.step([g.copy()])
        assert np.all(opt.state[0]["error"] == 0)
        assert np.allclose(p, tp.detach().numpy(), rtol=1e-5, atol=2e-7), t


def test_window_ages_past_the_ring_wrap_follow_the_gradient_history(oracle):
    """Which age a ring row gets once the ring has wrapped, pinned without the row formula:
    with k_init = 1 every gradient is kept whole in the row its step wrote, so at step t the
    update must be the sliding-window Adam direction over the last min(t, m) GRADIENTS, the
    newest with weight beta^0 and the one from j steps ago with beta^j, whatever rows they
    lie in.  A wrap in the wrong direction (ages counted from the wrong end of the ring, or an
    off-by-one at the write slot) changes the weights of all rows and fails from t = m + 1 on.
    t runs to 3 m + 2, three times round the ring."""
    rng = np.random.default_rng(5)
    d, m, lr, b1, b2, eps = 700, 5, 1e-2, 0.9, 0.999, 1e-8
    p = (rng.standard_normal(d) * 0.1).astype(np.float32)
    opt = oracle.OracleMicroAdam([p], m=m, lr=lr, quant_block_size=64, k_init=1.0,
                                 d_block_size=256)
    history = []
    worst = 0.0
    for t in range(1, 3 * m + 3):
        g = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.standard_normal(d).astype(np.float32)))
        history.append(g.astype(np.float64))
        before = p.astype(np.float64)
        opt.step([g.copy()])
        assert np.all(opt.state[0]["error"] == 0)
        assert opt.state[0]["index"] == t % m
        z1 = np.zeros(d)
        z2 = np.zeros(d)
        for j, gj in enumerate(reversed(history[-m:])):  # j steps ago
            z1 += b1 ** j * gj
            z2 += b2 ** j * gj ** 2
        want = ((1 - b1) * z1 / (1 - b1 ** t)) / (eps + np.sqrt((1 - b2) * z2 / (1 - b2 ** t)))
        got = (before - p.astype(np.float64)) / lr
        # p is fp32 of size ~0.1 (ulp 7.5e-9), so a step's difference quotient carries ~1e-6
        err = np.abs(got - want).max()
        worst = max(worst, err)
        assert err < 5e-6, (t, err)
        # and the wrong direction is far outside that tolerance once the ring has wrapped
        if t > m:
            z1w = sum(b1 ** (m - 1 - j) * gj for j, gj in enumerate(reversed(history[-m:])))
            wrong = ((1 - b1) * z1w / (1 - b1 ** t)) / (eps + np.sqrt((1 - b2) * z2 / (1 - b2 ** t)))
            assert np.abs(wrong - want).max() > 1e-2
    assert worst > 0.0


# ---- parameter update ------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_param_update_and_decay_against_torch(oracle, dtype):
    g = torch.Generator().manual_seed(3)
    p = (torch.randn(10000, generator=g) * 0.02).to(dtype)
    u = torch.randn(10000, generator=g).to(dtype)
    u[::3] = 0
    lr, wd = 1e-3, 0.1
    pa = bits(p)
    oracle.weight_decay(pa, np.float32(1 - lr * wd))
    p.mul_(1 - lr * wd)
    assert np.array_equal(pa, bits(p))
    oracle.param_update(pa, bits(u), np.float32(-lr))
    want = (p.float() + torch.tensor(-lr, dtype=torch.float32) * u.float()).to(dtype)
    assert np.array_equal(pa, bits(want))
    # torch's own add_(alpha=) may fuse the multiply-add; it stays within one ulp of p
    scale = p.double().abs() + lr * u.double().abs()
    p.add_(u, alpha=-lr)
    diff = (from_bits(pa).double() - p.double()).abs()
    ulp = scale * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -22) + 1e-30
    assert torch.all(diff <= ulp)


# ---- whole step, against the torch restatement ---------------------------------------------------

CASES = [
    # d list, dtype, m, q, k_init, alpha, wd, DB, steps
    ([3000, 257, 64, 1024], torch.bfloat16, 4, 64, 0.01, 0.0, 0.0, 1024, 9),
    ([5000], torch.float32, 3, 64, 0.02, 0.0, 0.0, 2048, 7),
    ([2500, 130], torch.bfloat16, 5, 32, 0.05, 0.0, 0.1, 512, 8),
    ([4100, 33], torch.bfloat16, 3, 1000, 0.01, 0.5, 0.0, 1024, 7),
    ([999], torch.float32, 2, 100, 0.03, 0.25, 0.01, 400, 5),
    ([3000, 257], torch.bfloat16, 4, 64, 0.01, -2, 0.0, 1024, 6),     # micro_adam.py:238-273
    ([1500], torch.float32, 3, 64, 0.02, -2, 0.05, 512, 5),
]


@pytest.mark.parametrize("sizes,dtype,m,q,k_init,alpha,wd,DB,steps", CASES)
def test_whole_step_matches_torch_restatement(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB,
                                              steps):
    gen = torch.Generator().manual_seed(0)
    params = [(torch.randn(n, generator=gen) * 0.02).to(dtype) for n in sizes]
    tref = TorchMicroAdam([p.clone() for p in params], m, 1e-3, q, k_init, alpha,
                          weight_decay=wd, d_block_size=DB)
    oparams = [bits(p) for p in params]
    oref = oracle.OracleMicroAdam(oparams, m, 1e-3, q, k_init, alpha, weight_decay=wd,
                                  d_block_size=DB)
    for s in range(steps):
        grads = [(torch.randn(n, generator=gen) * 0.01).to(dtype) for n in sizes]
        if s == 2:
            grads[0].zero_()  # an all-zero gradient: ties everywhere
        tref.step([g.clone() for g in grads])
        oref.step([bits(g) for g in grads])
        for i in range(len(sizes)):
            ts, os_ = tref.state[i], oref.state[i]
            assert ts["index"] == os_["index"]
            assert np.array_equal(ts["I"].numpy(), os_["I"]), (s, i)
            assert np.array_equal(bits(ts["V"]), os_["V"].reshape(ts["V"].shape)), (s, i)
            assert np.array_equal(ts["error"].numpy(), os_["error"]), (s, i)
            assert np.array_equal(bits(ts["min_vals"]), os_["min_vals"]), (s, i)
            assert np.array_equal(bits(ts["max_vals"]), os_["max_vals"]), (s, i)
            assert np.array_equal(bits(tref.params[i]), oparams[i]), (s, i)
            if alpha == -2:  # st['quant_err'] = a - Qinv(e_new), micro_adam.py:258-271
                assert np.array_equal(bits(ts["quant_err"]), os_["quant_err"]), (s, i)
                assert os_["quant_err"].any()


@pytest.mark.parametrize("sizes,dtype,m,q,k_init,alpha,wd,DB,steps", CASES)
def test_logged_sums_match_torch_restatement(oracle, sizes, dtype, m, q, k_init, alpha, wd, DB,
                                             steps):
    """The six sums of a logging step (micro_adam.py:155-156, :271-272, :306-308, :320-324)
    against the same sums taken with torch at the same points of the restated step.  Both sum
    the same values in float64; only the order of the additions differs (1e-12 relative).
    Placement matters and is what this pins: |u|^2 includes alpha * Qinv(e), the error norm is
    of the error feedback after the step's last requantisation, |g|^2 of the untouched
    gradient."""
    gen = torch.Generator().manual_seed(1)
    params = [(torch.randn(n, generator=gen) * 0.02).to(dtype) for n in sizes]
    tref = TorchMicroAdam([p.clone() for p in params], m, 1e-3, q, k_init, alpha,
                          weight_decay=wd, d_block_size=DB)
    oref = oracle.OracleMicroAdam([bits(p) for p in params], m, 1e-3, q, k_init, alpha,
                                  weight_decay=wd, d_block_size=DB)
    seen_nonzero = set()
    for s in range(steps):
        grads = [(torch.randn(n, generator=gen) * 0.01).to(dtype) for n in sizes]
        want = tref.step([g.clone() for g in grads], metrics=True)
        got = oref.step([bits(g) for g in grads], metrics=True)
        assert set(got) == set(want)
        for key in want:
            assert got[key] == pytest.approx(want[key], rel=1e-12, abs=0), (s, key)
            if want[key] != 0:
                seen_nonzero.add(key)
    expect = {"norm_g", "norm_u", "norm_e"}
    if alpha <= 0:
        expect |= {"sparsity_u"}  # (alpha > 0 makes the update dense)
    if alpha == -2:
        expect |= {"norm_qe"}
    assert expect <= seen_nonzero
    # a step without metrics moves the state exactly as one with them
    a = oracle.OracleMicroAdam([bits(p) for p in params], m, 1e-3, q, k_init, alpha,
                               weight_decay=wd, d_block_size=DB)
    b = oracle.OracleMicroAdam([bits(p) for p in params], m, 1e-3, q, k_init, alpha,
                               weight_decay=wd, d_block_size=DB)
    for s in range(3):
        grads = [bits((torch.randn(n, generator=gen) * 0.01).to(dtype)) for n in sizes]
        assert a.step([g.copy() for g in grads]) is None
        b.step([g.copy() for g in grads], metrics=True)
        for i in range(len(sizes)):
            assert np.array_equal(a.params[i], b.params[i])
            assert np.array_equal(a.state[i]["error"], b.state[i]["error"])


def test_error_feedback_invariant(oracle):
    """a_t = g_t + Qinv(e_t); after the step Qinv(e_{t+1}) reproduces a_t with the top-k
    entries removed, to within half a quantisation step."""
    rng = np.random.default_rng(4)
    d, q, DB = 4096, 64, 1024
    p = np.zeros(d, dtype=np.float32)
    opt = oracle.OracleMicroAdam([p], m=3, lr=1e-3, quant_block_size=q, k_init=0.01, d_block_size=DB)
    prev = np.zeros(d, dtype=np.float32)
    for t in range(5):
        g = (rng.standard_normal(d) * 1e-2).astype(np.float32)
        a = g + prev
        opt.step([g.copy()])
        st = opt.state[0]
        row = (st["index"] - 1) % 3
        pos = (np.arange(st["k"]) // st["k_block_size_many"]) * DB + st["I"][row]
        resid = a.copy()
        resid[pos] = 0
        deq = np.zeros(d, dtype=np.float32)
        oracle.asymm_block_quant_inv(d, q, st["error"], st["min_vals"], st["max_vals"], deq, 1.0)
        b = np.arange(d) // q
        u = (oracle.bf16_to_f32(st["max_vals"])[b] - oracle.bf16_to_f32(st["min_vals"])[b]) / 15
        # bf16 stats on fp32 data: allow the stats' own rounding on top of u/2
        slack = np.maximum(np.abs(oracle.bf16_to_f32(st["max_vals"])[b]),
                           np.abs(oracle.bf16_to_f32(st["min_vals"])[b])) * 2.0 ** -8
        assert np.all(np.abs(deq - resid) <= u / 2 + slack + 1e-9)
        # the kept entries are the largest in magnitude
        for blk in range(4):
            sel = st["I"][row][blk * st["k_block_size_many"]:(blk + 1) * st["k_block_size_many"]]
            blk_a = np.abs(a[blk * DB:(blk + 1) * DB])
            rest = np.delete(blk_a, sel)
            assert blk_a[sel].min() >= rest.max()
        prev = deq


# ---- Sparse M-FAC's window kernels: scalar products and linear combination -----------------

def _random_window(rng, d, dbs, k_init, m, values_f32):
    """A window in MicroAdam's layout whose rows name distinct coordinates per top-k block."""
    import math
    full, tail0 = d // dbs, (d // dbs) * dbs
    if d < dbs:
        full, tail0 = 1, d  # tools.py:85-92
    kb = math.ceil(min(dbs, d) * k_init)
    lens = [min(dbs, d)] * full + ([d - tail0] if tail0 < d else [])
    kbs = [kb] * full + ([math.ceil((d - tail0) * k_init)] if tail0 < d else [])
    k = sum(kbs)
    I = np.zeros((m, k), dtype=np.int16)
    for r in range(m):
        col = 0
        for ln, kk in zip(lens, kbs):
            I[r, col:col + kk] = rng.permutation(ln)[:kk]
            col += kk
    Vf = rng.standard_normal((m, k)).astype(np.float32)
    return I, Vf, k, kb


def _dense_rows(I, Vf, d, dbs, kb):
    """The window as a dense [m, d] float64 matrix (numpy fancy indexing, no oracle code)."""
    m, k = I.shape
    pos = (np.arange(k) // kb) * dbs + I.astype(np.int64)
    G = np.zeros((m, d))
    G[np.arange(m)[:, None], pos] = Vf
    return G


@pytest.mark.parametrize("values_f32", [False, True])
@pytest.mark.parametrize("d,dbs,k_init", [(1000, 256, 0.05), (4096, 512, 0.01), (300, 512, 0.1),
                                          (2048 + 7, 1024, 0.02)])
def test_sparse_scalar_products_equal_dense_matvec(oracle, values_f32, d, dbs, k_init):
    rng = np.random.default_rng(d)
    m = 6
    I, Vf, k, kb = _random_window(rng, d, dbs, k_init, m, values_f32)
    V = Vf if values_f32 else oracle.f32_to_bf16(Vf)
    Vw = Vf if values_f32 else oracle.bf16_to_f32(V)
    gf = rng.standard_normal(d).astype(np.float32)
    g = gf if values_f32 else oracle.f32_to_bf16(gf)
    gw = gf if values_f32 else oracle.bf16_to_f32(g)
    rows = 4  # the last two rows of the window are not live
    out = np.full(m, 0.5)
    oracle.sparse_scalar_products(d, rows, k, dbs, kb, g, I, V, out)
    want = _dense_rows(I, Vw, d, dbs, kb) @ gw.astype(np.float64)
    assert np.allclose(out[:rows], 0.5 + want[:rows], rtol=1e-12, atol=1e-12)
    assert np.all(out[rows:] == 0.5)


@pytest.mark.parametrize("out_f32", [False, True])
@pytest.mark.parametrize("d,dbs,k_init", [(1000, 256, 0.05), (300, 512, 0.1), (2048 + 7, 1024, 0.5)])
def test_sparse_linear_combination_equals_dense_combination(oracle, out_f32, d, dbs, k_init):
    rng = np.random.default_rng(d + 1)
    m = 7
    I, Vf, k, kb = _random_window(rng, d, dbs, k_init, m, True)
    V = oracle.f32_to_bf16(Vf)
    Vw = oracle.bf16_to_f32(V)
    coef = rng.standard_normal(m).astype(np.float32)
    rows = 5
    out = np.zeros(d, dtype=np.float32) if out_f32 else np.zeros(d, dtype=np.uint16)
    oracle.sparse_linear_combination(d, rows, k, dbs, kb, coef, I, V, out)
    got = out if out_f32 else oracle.bf16_to_f32(out)
    G = _dense_rows(I, Vw, d, dbs, kb)
    want = coef[:rows].astype(np.float64) @ G[:rows]
    scale = np.abs(coef[:rows]).astype(np.float64) @ np.abs(G[:rows])
    tol = (2.0 ** -22 if out_f32 else 2.0 ** -8) * scale + 1e-30
    assert np.all(np.abs(got - want) <= tol)
    assert np.all(got[scale == 0] == 0)


def test_sparse_linear_combination_special_cases(oracle):
    """One row with coefficient 1 is copy_values k2d; disjoint rows give the exact products;
    the result is added to what out holds."""
    rng = np.random.default_rng(5)
    d, dbs, m = 1536, 512, 3
    I, Vf, k, kb = _random_window(rng, d, dbs, 0.03, m, True)
    V = oracle.f32_to_bf16(Vf)
    out = np.zeros(d, dtype=np.uint16)
    oracle.sparse_linear_combination(d, 1, k, dbs, kb, np.ones(1, np.float32), I, V, out)
    scat = np.zeros(d, dtype=np.uint16)
    oracle.copy_values(d, k, dbs, kb, I[0], V[0], scat, 0)
    assert np.array_equal(out, scat)
    # rows on disjoint coordinates: every touched coordinate is one product, rounded once
    I2 = I.copy()
    for b in range(d // dbs):
        perm = rng.permutation(dbs)[:m * kb].reshape(m, kb)
        I2[:, b * kb:(b + 1) * kb] = perm
    coef = np.array([0.5, -3.0, 1.25], dtype=np.float32)
    out = np.full(d, 2.0, dtype=np.float32)
    oracle.sparse_linear_combination(d, m, k, dbs, kb, coef, I2, V, out)
    want = np.full(d, 2.0, dtype=np.float32)
    pos = (np.arange(k) // kb) * dbs + I2.astype(np.int64)
    for r in range(m):
        want[pos[r]] = np.float32(2.0) + coef[r] * oracle.bf16_to_f32(V[r])
    assert np.array_equal(out, want)
