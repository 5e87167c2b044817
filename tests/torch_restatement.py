"""Second, independent CPU statement of the MicroAdam step, in stock torch ops.

Used only by the tests, to pin the C oracle: both follow
ista_daslab_optimizers/micro_adam/micro_adam.py:146-328 op for op, but this one leans
on torch's own kernels (abs, stable sort, min, max, add_, mul_, dtype casts) for every
piece of arithmetic and rounding that torch defines, so an indexing or rounding slip in
the C file shows up as a bit difference.  The five extension ops the reference calls
into are written out here with torch tensor arithmetic in fp32.
"""
import math

import numpy as np
import torch


def block_split(n, b):
    if n < b:
        return 1, n
    return int(n / b), n - n % b


def topk_lowest_index(x_abs_2d, k):
    """Indices of the k largest per row, ties to the lowest index, ascending order."""
    order = torch.sort(x_abs_2d.float(), dim=1, descending=True, stable=True).indices[:, :k]
    return torch.sort(order, dim=1).values


def unpack(xq, d):
    hi = (xq >> 4).to(torch.float32)
    lo = (xq & 0x0F).to(torch.float32)
    return torch.stack((hi, lo), dim=1).reshape(-1)[:d]


def block_ids(d, q):
    return torch.arange(d, dtype=torch.int64) // q


def qinv_accumulate(d, q, xq, xmin, xmax, x, alpha):
    b = block_ids(d, q)
    mn = xmin.float()[b]
    mx = xmax.float()[b]
    u = (mx - mn) / 15.0
    deq = unpack(xq, d) * u
    deq = deq + mn
    add = torch.tensor(alpha, dtype=torch.float32) * deq
    x.copy_((x.float() + add).to(x.dtype))


def quantize(d, q, xq, xmin, xmax, x):
    b = block_ids(d, q)
    mn = xmin.float()[b]
    mx = xmax.float()[b]
    u = (mx - mn) / 15.0
    ok = (u != 0) & torch.isfinite(u)
    v = torch.floor((x.float() - mn) / u + 0.5)
    v = torch.where(torch.isnan(v), torch.zeros_like(v), v).clamp(0, 15)
    codes = torch.where(ok, v, torch.zeros_like(v)).to(torch.uint8)
    if d % 2:
        codes = torch.cat((codes, torch.zeros(1, dtype=torch.uint8)))
    xq.copy_((codes[0::2] << 4) | codes[1::2])


class TorchMicroAdam:
    def __init__(self, params, m, lr, quant_block_size, k_init=0.01, alpha=0, betas=(0.9, 0.999),
                 weight_decay=0, eps=1e-8, d_block_size=20480):
        self.params = [p.view(-1) for p in params]
        self.m, self.lr, self.q = m, lr, int(quant_block_size)
        self.k_init, self.alpha, self.wd = k_init, alpha, weight_decay
        self.beta1, self.beta2, self.eps = betas[0], betas[1], eps
        self.DB = d_block_size
        self.steps = 0
        self.state = [None] * len(self.params)

    def _init(self, i):
        d = self.params[i].numel()
        st = {}
        st["dbs"] = d if d < self.DB else self.DB
        st["full"], st["d_index_topk"] = block_split(d, st["dbs"])
        st["k_many"] = int(math.ceil(st["dbs"] * self.k_init))
        st["k_few"] = int(math.ceil((d - st["d_index_topk"]) * self.k_init))
        st["k_index"] = st["full"] * st["k_many"]
        st["k"] = st["k_index"] + st["k_few"]
        st["index"] = 0
        st["I"] = torch.zeros(self.m, st["k"], dtype=torch.int16)
        st["V"] = torch.zeros(self.m, st["k"], dtype=torch.bfloat16)
        st["qfull"], st["d_index_quant"] = block_split(d, self.q)
        st["error"] = torch.zeros(int(math.ceil(d / 2)), dtype=torch.uint8)
        st["min_vals"] = torch.zeros(st["qfull"] + 1, dtype=torch.bfloat16)
        st["max_vals"] = torch.zeros(st["qfull"] + 1, dtype=torch.bfloat16)
        self.state[i] = st
        return st

    def _stats(self, st, grad, d):
        qf, diq = st["qfull"], st["d_index_quant"]
        if qf == 1:
            st["min_vals"][:1] = grad[:diq].min()
            st["max_vals"][:1] = grad[:diq].max()
        else:
            st["min_vals"][:qf] = grad[:diq].view(qf, self.q).min(dim=1).values
            st["max_vals"][:qf] = grad[:diq].view(qf, self.q).max(dim=1).values
        if diq < d:
            st["min_vals"][qf] = grad[diq:].min()
            st["max_vals"][qf] = grad[diq:].max()

    def _adam_direction(self, st, grad, d):
        t, m = self.steps, self.m
        rows = min(t, m)
        z1 = torch.zeros(d, dtype=torch.float32)
        z2 = torch.zeros(d, dtype=torch.float32)
        hit = torch.zeros(d, dtype=torch.bool)
        j = torch.arange(st["k"], dtype=torch.int64)
        base = (j // st["k_many"]) * st["dbs"]
        for r in range(rows):
            age = (t - 1 - r) % m
            w1 = torch.tensor(float(self.beta1) ** age, dtype=torch.float32)
            w2 = torch.tensor(float(self.beta2) ** age, dtype=torch.float32)
            pos = base + st["I"][r].to(torch.int64)
            v = st["V"][r].float()
            z1[pos] = z1[pos] + w1 * v
            z2[pos] = z2[pos] + w2 * (v * v)
            hit[pos] = True
        s1 = torch.tensor((1 - self.beta1) / (1 - self.beta1 ** t), dtype=torch.float32)
        s2 = torch.tensor((1 - self.beta2) / (1 - self.beta2 ** t), dtype=torch.float32)
        # torch's vectorised CPU sqrt is not correctly rounded in this build (about 0.6 % of
        # fp32 inputs are one ulp off); numpy's is IEEE, as sqrtf is
        root = torch.from_numpy(np.sqrt((z2 * s2).numpy()))
        out = (z1 * s1) / (torch.tensor(self.eps, dtype=torch.float32) + root)
        grad[hit] = out[hit].to(grad.dtype)

    def step(self, grads, lr=None, metrics=False):
        """metrics=True: also the sums of a logging step, taken with torch at the points of
        micro_adam.py:155-156, :258-273, :306-308, :320-324 (in float64, from the buffers as they
        are at that point)."""
        self.steps += 1
        lr = self.lr if lr is None else lr
        sums = dict(norm_qe=0.0, norm_g=0.0, norm_u=0.0, norm_e=0.0, sparsity_u=0.0, sparsity_qe=0.0)

        def sq(x):
            return float(x.double().pow(2).sum())

        for i, (p, grad) in enumerate(zip(self.params, grads)):
            if grad is None:
                continue
            grad = grad.view(-1)
            d = p.numel()
            sums["norm_g"] += sq(grad)
            st = self.state[i] or self._init(i)
            index, I, V = st["index"], st["I"], st["V"]
            dbs, full, dit = st["dbs"], st["full"], st["d_index_topk"]
            qinv_accumulate(d, self.q, st["error"], st["min_vals"], st["max_vals"], grad, 1.0)
            I[index, :st["k_index"]] = topk_lowest_index(
                grad[:dit].abs().view(full, dbs), st["k_many"]).to(torch.int16).view(-1)
            if st["k_few"] > 0:
                I[index, st["k_index"]:] = topk_lowest_index(
                    grad[dit:].abs().view(1, -1), st["k_few"]).to(torch.int16).view(-1)
            j = torch.arange(st["k"], dtype=torch.int64)
            pos = (j // st["k_many"]) * dbs + I[index].to(torch.int64)
            V[index, :] = grad[pos].to(torch.bfloat16)
            st["index"] = (index + 1) % self.m
            grad[pos] = 0
            self._stats(st, grad, d)
            quantize(d, self.q, st["error"], st["min_vals"], st["max_vals"], grad)
            if self.wd > 0:
                p.mul_(1 - lr * self.wd)
            if self.alpha == -2:
                # micro_adam.py:258-273: p = p - a, then p = p + Qinv(e_new); quant_err = a - Qinv(e_new)
                quant_err = st["quant_err"] = torch.zeros_like(p).view(-1)
                quant_err.add_(grad)
                p.add_(grad, alpha=-1)
                grad.zero_()
                qinv_accumulate(d, self.q, st["error"], st["min_vals"], st["max_vals"], grad, 1.0)
                p.add_(grad)
                quant_err.sub_(grad)
                sums["norm_qe"] += sq(quant_err)
                sums["sparsity_qe"] += float((quant_err == 0).sum())
            grad.zero_()
            self._adam_direction(st, grad, d)
            if self.alpha > 0:
                qinv_accumulate(d, self.q, st["error"], st["min_vals"], st["max_vals"], grad,
                                self.alpha)
            p.copy_((p.float() + torch.tensor(-lr, dtype=torch.float32) * grad.float()).to(p.dtype))
            sums["norm_u"] += sq(grad)
            sums["sparsity_u"] += float((grad == 0).sum())
            if self.alpha > 0:
                grad.zero_()
                qinv_accumulate(d, self.q, st["error"], st["min_vals"], st["max_vals"], grad,
                                1 - self.alpha)
                self._stats(st, grad, d)
                quantize(d, self.q, st["error"], st["min_vals"], st["max_vals"], grad)
            if metrics:
                grad.zero_()
                qinv_accumulate(d, self.q, st["error"], st["min_vals"], st["max_vals"], grad, 1.0)
                sums["norm_e"] += sq(grad)
        return sums if metrics else None
