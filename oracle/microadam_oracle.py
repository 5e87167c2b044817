"""ctypes front end of the CPU oracle (oracle/microadam_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The shipped package never imports this module.

bf16 data is carried as numpy uint16 arrays (the raw bit patterns); fp32 data as
numpy float32 arrays.  `OracleMicroAdam` mirrors the constructor of the reference's
MicroAdam (ista_daslab_optimizers/micro_adam/micro_adam.py:14) and its state keys
(:61-94) on numpy arrays.
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmicroadam_oracle.so")

F32, BF16 = 0, 1


def build(force=False):
    """Compile the oracle with gcc (a few hundred ms)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
            os.path.join(_HERE, "microadam_oracle.c")):
        subprocess.check_call(["make", "-s", "-C", _HERE, "-B"])
    return _SO


class _Geom(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in (
        "d", "d_block_size", "topk_full_blocks_count", "d_index_topk", "k_block_size_many",
        "k_block_size_few", "k_index", "k", "quant_full_blocks_count", "d_index_quant",
        "error_bytes", "stats_len")]


class _Hyper(ctypes.Structure):
    _fields_ = [("t", ctypes.c_int64), ("m", ctypes.c_int64), ("q", ctypes.c_int64),
                ("max_d_block_size", ctypes.c_int64), ("k_init", ctypes.c_double),
                ("alpha", ctypes.c_double), ("beta1", ctypes.c_double),
                ("beta2", ctypes.c_double), ("eps", ctypes.c_double), ("lr", ctypes.c_double),
                ("wd", ctypes.c_double)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        vp, i64, f32, f64, ci = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_float,
                                 ctypes.c_double, ctypes.c_int)
        L.ora_set_threads.argtypes = [ci]
        L.ora_get_threads.restype = ci
        L.ora_f32_to_bf16.argtypes = [f32]
        L.ora_f32_to_bf16.restype = ctypes.c_uint16
        L.ora_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.ora_bf16_to_f32.restype = f32
        L.ora_block_split.argtypes = [i64, i64, ctypes.POINTER(i64), ctypes.POINTER(i64)]
        L.ora_geometry.argtypes = [i64, i64, f64, i64, ctypes.POINTER(_Geom)]
        L.ora_asymm_block_quant_inv.argtypes = [i64, i64, vp, vp, vp, vp, f32, ci]
        L.ora_asymm_block_quant.argtypes = [i64, i64, vp, vp, vp, vp, ci]
        L.ora_block_minmax.argtypes = [i64, i64, vp, ci, vp, vp]
        L.ora_block_topk.argtypes = [i64, i64, i64, i64, vp, ci, vp]
        L.ora_copy_values.argtypes = [i64, i64, i64, i64, vp, vp, vp, ci, ci]
        L.ora_zerorize_block_components.argtypes = [vp, vp, i64, i64, i64, i64, ci]
        L.ora_compute_microadam_update.argtypes = [i64, f64, f64, f64, i64, i64, i64, i64, i64,
                                                   vp, vp, vp, ci]
        L.ora_weight_decay.argtypes = [i64, vp, f32, ci]
        L.ora_param_update.argtypes = [i64, vp, vp, f32, ci, ci]
        L.ora_update_step.argtypes = [ctypes.POINTER(_Hyper), vp, vp, ci, i64,
                                      ctypes.POINTER(i64), vp, vp, vp, vp, vp]
        L.ora_update_step.restype = ci
        L.ora_step_metrics.argtypes = L.ora_update_step.argtypes + [ctypes.POINTER(f64)]
        L.ora_step_metrics.restype = ci
        L.ora_update_step_state.argtypes = L.ora_step_metrics.argtypes + [vp]
        L.ora_update_step_state.restype = ci
        L.ora_sparse_scalar_products.argtypes = [i64, i64, i64, i64, i64, vp, ci, vp, vp, ci, vp]
        L.ora_sparse_linear_combination.argtypes = [i64, i64, i64, i64, i64, vp, vp, vp, ci, vp,
                                                    ci]
        _lib = L
    return _lib


def _ptr(a):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


def dtype_tag(a):
    if a.dtype == np.float32:
        return F32
    if a.dtype == np.uint16:
        return BF16
    raise TypeError(f"oracle arrays are float32 or uint16 (bf16 bits), got {a.dtype}")


# ---- bf16 helpers on numpy arrays -------------------------------------------

def bf16_to_f32(h):
    return (np.asarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(f):
    """Round-to-nearest-even narrowing of a float32 array to bf16 bit patterns."""
    u = np.ascontiguousarray(f, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x0040).astype(np.uint16)
    return r


# ---- thin per-op wrappers ------------------------------------------------------

def set_threads(n):
    lib().ora_set_threads(int(n))


def get_threads():
    return int(lib().ora_get_threads())


def block_split(n, b):
    c, s = ctypes.c_int64(), ctypes.c_int64()
    lib().ora_block_split(n, b, ctypes.byref(c), ctypes.byref(s))
    return c.value, s.value


def geometry(d, max_d_block_size, k_init, q):
    g = _Geom()
    lib().ora_geometry(d, max_d_block_size, float(k_init), q, ctypes.byref(g))
    return {n: getattr(g, n) for n, _ in _Geom._fields_}


def asymm_block_quant_inv(d, q, xq, xmin, xmax, x, alpha):
    lib().ora_asymm_block_quant_inv(d, q, _ptr(xq), _ptr(xmin), _ptr(xmax), _ptr(x), float(alpha),
                                    dtype_tag(x))


def asymm_block_quant(d, q, xq, xmin, xmax, x):
    lib().ora_asymm_block_quant(d, q, _ptr(xq), _ptr(xmin), _ptr(xmax), _ptr(x), dtype_tag(x))


def block_minmax(d, q, x, xmin, xmax):
    lib().ora_block_minmax(d, q, _ptr(x), dtype_tag(x), _ptr(xmin), _ptr(xmax))


def block_topk(d, d_block_size, k_many, k_few, x, I_row):
    lib().ora_block_topk(d, d_block_size, k_many, k_few, _ptr(x), dtype_tag(x), _ptr(I_row))


def copy_values(d, k, d_block_size, k_block_size, indices, inp, out, direction):
    tag = dtype_tag(inp) if direction == 1 else dtype_tag(out)
    if direction != 1 and out.dtype == np.uint16 and inp.dtype != np.uint16:
        raise TypeError("k2d takes bf16 values")
    lib().ora_copy_values(d, k, d_block_size, k_block_size, _ptr(indices), _ptr(inp), _ptr(out),
                          direction, tag)


def zerorize_block_components(vector, indices, d, k, d_block_size, k_block_size):
    lib().ora_zerorize_block_components(_ptr(vector), _ptr(indices), d, k, d_block_size,
                                        k_block_size, dtype_tag(vector))


def compute_microadam_update(t, beta1, beta2, eps, d_block_size, k_block_size, d, m, k, indices,
                             values, out):
    lib().ora_compute_microadam_update(t, beta1, beta2, eps, d_block_size, k_block_size, d, m, k,
                                       _ptr(indices), _ptr(values), _ptr(out), dtype_tag(out))


def weight_decay(p, factor):
    lib().ora_weight_decay(p.size, _ptr(p), float(factor), dtype_tag(p))


def param_update(p, u, neg_lr):
    lib().ora_param_update(p.size, _ptr(p), _ptr(u), float(neg_lr), dtype_tag(p), dtype_tag(u))


def sparse_scalar_products(d, m_rows, k, d_block_size, k_block_size, g, indices, values, out):
    """out (float64, length >= m_rows) += scalar products of the window rows with g."""
    assert out.dtype == np.float64
    lib().ora_sparse_scalar_products(d, m_rows, k, d_block_size, k_block_size, _ptr(g),
                                     dtype_tag(g), _ptr(indices), _ptr(values), dtype_tag(values),
                                     _ptr(out))


def sparse_linear_combination(d, m_rows, k, d_block_size, k_block_size, coef, indices, values,
                              out):
    """out += sum_i coef[i] * (window row i scattered to length d)."""
    assert coef.dtype == np.float32
    lib().ora_sparse_linear_combination(d, m_rows, k, d_block_size, k_block_size, _ptr(coef),
                                        _ptr(indices), _ptr(values), dtype_tag(values), _ptr(out),
                                        dtype_tag(out))


def unpack_codes(xq, d):
    """4-bit codes of a packed error buffer, element 2j in the high nibble of byte j."""
    xq = np.asarray(xq, dtype=np.uint8)
    out = np.empty(xq.size * 2, dtype=np.uint8)
    out[0::2] = xq >> 4
    out[1::2] = xq & 0x0F
    return out[:d]


def canonical_window(I, V, k_block_size_many):
    """Window rows with the entries of every block sorted by index.

    The order of the k_block entries inside a block of a row carries no meaning (the reference
    takes them from torch.topk(sorted=False), micro_adam.py:193-200, and the Adam statistics do
    not depend on it), so two states are the same window iff they agree after this sort."""
    I = np.asarray(I)
    V = np.asarray(V).reshape(I.shape)
    blk = (np.arange(I.shape[1]) // k_block_size_many).astype(np.int64)
    key = blk[None, :] * 65536 + I.astype(np.int64)
    order = np.argsort(key, axis=1, kind="stable")
    return np.take_along_axis(I, order, axis=1), np.take_along_axis(V, order, axis=1)


# ---- optimizer-shaped driver -----------------------------------------------------

class OracleMicroAdam:
    """MicroAdam on numpy arrays; constructor arguments as micro_adam.py:14.

    `params` is a list of 1-D-viewable numpy arrays (float32, or uint16 holding bf16 bits)
    updated in place; `step(grads)` consumes the gradient arrays as scratch, like the
    reference does with p.grad (micro_adam.py:153).  `d_block_size` is the top-k block
    size the reference derives from the device's shared memory (:43-44).
    """

    def __init__(self, params, m, lr, quant_block_size, k_init=0.01, alpha=0, betas=(0.9, 0.999),
                 weight_decay=0, eps=1e-8, d_block_size=20480):
        assert (0 <= alpha < 1) or alpha == -2
        self.params = [p.reshape(-1) for p in params]
        self.m, self.lr, self.quant_block_size = m, lr, int(quant_block_size)
        self.k_init, self.alpha, self.weight_decay = k_init, alpha, weight_decay
        self.beta1, self.beta2, self.eps = betas[0], betas[1], eps
        self.d_block_size = d_block_size
        self.steps = 0
        self.state = [None] * len(self.params)

    def _init_state(self, i):
        p = self.params[i]
        g = geometry(p.size, self.d_block_size, self.k_init, self.quant_block_size)
        st = dict(g)
        st["index"] = 0
        st["I"] = np.zeros((self.m, g["k"]), dtype=np.int16)
        st["V"] = np.zeros((self.m, g["k"]), dtype=np.uint16)
        st["error"] = np.zeros(int(math.ceil(p.size / 2)), dtype=np.uint8)
        st["min_vals"] = np.zeros(g["stats_len"], dtype=np.uint16)
        st["max_vals"] = np.zeros(g["stats_len"], dtype=np.uint16)
        if self.alpha == -2:  # micro_adam.py:67-68
            st["quant_err"] = np.zeros_like(p)
        self.state[i] = st
        return st

    METRICS = ("norm_qe", "norm_g", "norm_u", "norm_e", "sparsity_u", "sparsity_qe")

    def step(self, grads, lr=None, metrics=False):
        """One optimizer step.  metrics=True: a logging step (micro_adam.py:155-156, :271-272,
        :306-308, :320-324); returns the six sums over the tensors that the reference hands
        to its _log (:328, :330) as a dict of Python floats: squared norms and zero counts."""
        self.steps += 1
        lr = self.lr if lr is None else lr
        h = _Hyper(self.steps, self.m, self.quant_block_size, self.d_block_size, self.k_init,
                   float(self.alpha), self.beta1, self.beta2, self.eps, lr, self.weight_decay)
        sums = (ctypes.c_double * 6)()
        for i, (p, g) in enumerate(zip(self.params, grads)):
            if g is None:
                continue
            g = g.reshape(-1)
            assert g.dtype == p.dtype and g.size == p.size
            st = self.state[i] or self._init_state(i)
            idx = ctypes.c_int64(st["index"])
            args = (ctypes.byref(h), _ptr(p), _ptr(g), dtype_tag(p), p.size, ctypes.byref(idx),
                    _ptr(st["I"]), _ptr(st["V"]), _ptr(st["error"]), _ptr(st["min_vals"]),
                    _ptr(st["max_vals"]))
            qe = _ptr(st["quant_err"]) if "quant_err" in st else None
            rc = lib().ora_update_step_state(*args, sums if metrics else None, qe)
            if rc != 0:
                raise NotImplementedError("oracle covers alpha in [0, 1) and alpha == -2")
            st["index"] = idx.value
        return dict(zip(self.METRICS, sums)) if metrics else None
