"""Writes tests/golden/microadam_small.npz: inputs and expected outputs of a few small MicroAdam
runs, produced by the CPU oracle (oracle/microadam_oracle.c).

The reference holds no golden vectors for this path and its kernels cannot run here, so these
fixtures record the oracle's own answers once its pins (tests/test_oracle_pins.py) are green.
They guard the oracle against silent change and give the GPU tests inputs that do not depend
on a random-number generator's implementation.  Run from the repository root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
import microadam_oracle as oracle  # noqa: E402

CASES = {
    # name: (sizes, dtype, m, q, k_init, alpha, wd, d_block_size, steps)
    "bf16_q64": ([3000, 257, 1024], "bf16", 4, 64, 0.01, 0.0, 0.0, 1024, 6),
    "f32_q64_wd": ([4096], "f32", 3, 64, 0.02, 0.0, 0.01, 2048, 5),
    "bf16_alpha": ([2500, 33], "bf16", 3, 1000, 0.01, 0.5, 0.0, 1024, 5),
    "bf16_block20480": ([20480 + 4096], "bf16", 3, 64, 0.01, 0.0, 0.0, 20480, 4),
    # quantisation blocks longer than the top-k blocks, without and with alpha
    "bf16_longq": ([1024 * 5 + 77, 300], "bf16", 4, 2048, 0.02, 0.0, 0.0, 1024, 5),
    "bf16_longq_alpha": ([1024 * 5 + 77], "bf16", 4, 2048, 0.02, 0.3, 0.0, 1024, 5),
    "bf16_q64_alpha": ([3000, 1024], "bf16", 3, 64, 0.02, 0.5, 0.01, 1024, 5),
    "f32_alpha_minus2": ([2000], "f32", 3, 64, 0.02, -2, 0.0, 1024, 4),
}

# Sparse M-FAC's window kernels (scalar products, linear combination) on the final window of
# tensor 0 of a case above: name -> (case, live rows)
SPARSE_CASES = {
    "sparse_bf16_q64": ("bf16_q64", 4),
    "sparse_bf16_block20480": ("bf16_block20480", 2),
    "sparse_f32_q64_wd": ("f32_q64_wd", 3),
}


def main():
    out = {}
    rng = np.random.default_rng(20240613)
    for name, (sizes, dtype, m, q, k_init, alpha, wd, DB, steps) in CASES.items():
        def draw(n, std):
            x = (rng.standard_normal(n) * std).astype(np.float32)
            return oracle.f32_to_bf16(x) if dtype == "bf16" else x
        params = [draw(n, 0.02) for n in sizes]
        grads = [[draw(n, 0.01) for n in sizes] for _ in range(steps)]
        grads[1][0][:] = 0  # one all-zero gradient: ties everywhere
        for i, p in enumerate(params):
            out[f"{name}/p0/{i}"] = p.copy()
        opt = oracle.OracleMicroAdam(params, m, 1e-3, q, k_init, alpha, weight_decay=wd,
                                     d_block_size=DB)
        for s in range(steps):
            for i, g in enumerate(grads[s]):
                out[f"{name}/g/{s}/{i}"] = g.copy()
            opt.step([g.copy() for g in grads[s]])
        for i, p in enumerate(params):
            st = opt.state[i]
            I, V = oracle.canonical_window(st["I"], st["V"], st["k_block_size_many"])
            out[f"{name}/p/{i}"] = p.copy()
            out[f"{name}/I/{i}"] = I
            out[f"{name}/V/{i}"] = V
            out[f"{name}/error/{i}"] = st["error"].copy()
            out[f"{name}/min_vals/{i}"] = st["min_vals"].copy()
            out[f"{name}/max_vals/{i}"] = st["max_vals"].copy()
            out[f"{name}/index/{i}"] = np.int64(st["index"])
    rng2 = np.random.default_rng(20240614)  # its own stream: the arrays above stay as they were
    for name, (case, rows) in SPARSE_CASES.items():
        sizes, dtype, m, q, k_init, alpha, wd, DB, steps = CASES[case]
        d = sizes[0]
        geo = oracle.geometry(d, DB, k_init, q)
        I, V = out[f"{case}/I/0"], out[f"{case}/V/0"]
        if dtype == "f32":  # fp32 vectors go with fp32 values (use_bf16 = False)
            V = oracle.bf16_to_f32(V)
        g = rng2.standard_normal(d).astype(np.float32)
        g = oracle.f32_to_bf16(g) if dtype == "bf16" else g
        coef = rng2.standard_normal(m).astype(np.float32)
        dots = np.zeros(m)
        oracle.sparse_scalar_products(d, rows, geo["k"], geo["d_block_size"],
                                      geo["k_block_size_many"], g, I, V, dots)
        comb = np.zeros(d, dtype=g.dtype)
        oracle.sparse_linear_combination(d, rows, geo["k"], geo["d_block_size"],
                                         geo["k_block_size_many"], coef, I, V, comb)
        out[f"{name}/g"], out[f"{name}/coef"] = g, coef
        out[f"{name}/dots"], out[f"{name}/comb"] = dots, comb
    np.savez_compressed(os.path.join(HERE, "microadam_small.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
