"""MicroAdam step benchmark on one MI355X.

A "step" is one `optimizer.step()` over the whole parameter list of the workload, with
parameters, gradients and optimizer state already resident in HBM.  The default workload is the
Llama-2-7B-shaped list (6.74 B bf16 parameters, m=10, k=1 %, quant block 64, alpha=0).
Gradients are synthetic N(0, 1e-3^2) bf16, drawn on the device before the timed region; m + 2
distinct gradient sets are used in turn, so that no gradient recurs inside the window.

Prints ONE JSON line: params/s (whole job), ms per step, the HBM roofline of the fused step
kernel (algorithmic bytes per parameter x parameters / measured duration against 8 TB/s) and a
CPU baseline: the C oracle (a port of the reference's step; the reference has no CPU path)
timed on this host's cores over a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "ista-daslab-optimizers_amd"))

HBM_PEAK_GBS = 8000.0
CAL_BYTES = 26214 * 40960  # --copy-calibration: bytes the known-size copy reads (and writes), ~1 GiB

# HBM bytes per step from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same
# counters read for a plain copy of known size; (workload, op_by_op) -> bytes.  The figures and
# the commands behind them are in profiles/.
MEASURED_TRAFFIC = {
    ("llama2-7b", False): (50.596e9, "profiles/fused_step_llama2-7b_hbm_traffic.txt"),
    ("gpt2-small", False): (0.939e9, "profiles/fused_step_gpt2-small_hbm_traffic.txt"),
    ("outlier-1.3b", False): (15.743e9, "profiles/fused_step_outlier-1.3b_hbm_traffic.txt"),
    ("llama3-8b", False): (92.069e9, "profiles/spanning_step_llama3-8b_hbm_traffic.txt"),
    ("llama2-7b-q100k", False): (49.984e9, "profiles/spanning_step_llama2-7b-q100k_hbm_traffic.txt"),
}


def llama2_7b():
    shapes = [(32000, 4096)]
    for _ in range(32):
        shapes += [(4096, 4096)] * 4 + [(11008, 4096)] * 3 + [(4096,)] * 2
    shapes += [(32000, 4096)]
    return shapes


def gpt2_small():
    shapes = [(50257, 768), (1024, 768)]
    for _ in range(12):
        shapes += [(768,), (768,), (768, 2304), (2304,), (768, 768), (768,), (768,), (768,),
                   (768, 3072), (3072,), (3072, 768), (768,)]
    shapes += [(768,), (768,)]
    return shapes


def outlier_1p3b():
    shapes = [(50304, 2048)]
    for _ in range(24):
        shapes += [(2048, 6144), (2048, 2048), (2048, 8192), (8192, 2048)]
    return shapes


def llama3_8b():
    shapes = [(128256, 4096)]
    for _ in range(32):
        shapes += [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096)] + [(14336, 4096)] * 3
    shapes += [(128256, 4096)]
    return shapes


WORKLOADS = {
    # name: (shapes, dtype, m, k_init, q, alpha, grad_std)
    "llama2-7b": (llama2_7b, "bf16", 10, 0.01, 64, 0.0, 1e-3),
    "gpt2-small": (gpt2_small, "bf16", 10, 0.01, 64, 0.0, 1e-2),
    "outlier-1.3b": (outlier_1p3b, "bf16", 20, 0.05, 32, 0.0, 1e-3),
    "llama3-8b": (llama3_8b, "bf16", 10, 0.01, 100000, 0.5, 1e-3),
    "plumbing-1m": (lambda: [(1048576,)], "f32", 10, 0.01, 64, 0.0, 1.0),
    # not one of the five benchmark configurations: the 7B list with the quantisation block of the reference's
    # README (quant_block_size=100_000, alpha=0), which takes the two-pass route
    "llama2-7b-q100k": (llama2_7b, "bf16", 10, 0.01, 100000, 0.0, 1e-3),
    # not one of the five either: the 7B list with alpha > 0 and short quantisation blocks
    "llama2-7b-alpha": (llama2_7b, "bf16", 10, 0.01, 64, 0.5, 1e-3),
}


_probe = None


def stream_probe():
    """ma_stream_probe of libmicroadam_probe.so (csrc/stream_probe.h): known-size streaming
    kernels, measurement tooling that only this benchmark loads."""
    global _probe
    if _probe is None:
        import ctypes
        path = os.path.join(ROOT, "ista-daslab-optimizers_amd", "ista_daslab_optimizers",
                            "libmicroadam_probe.so")
        fn = ctypes.CDLL(path).ma_stream_probe
        vp = ctypes.c_void_p
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, vp, vp, vp, vp,
                       vp, vp]

        def call(*args):
            rc = fn(*args)
            if rc:
                raise RuntimeError(f"ma_stream_probe failed with code {rc}")
        _probe = call
    return _probe


def numel(shape):
    n = 1
    for s in shape:
        n *= s
    return n


def algorithmic_bytes_per_param(shapes, dtype, m, k_init, q, alpha, d_block_size, first_step,
                                n_steps):
    """Every array of the step touched once: read g, read+write 4-bit EF, read+write p, write
    one window row (int16 + bf16), read min(t, m) window rows, read+write bf16 min/max.
    Averaged over the timed steps t = first_step .. first_step + n_steps - 1 (a step with a
    window that is still filling reads fewer rows)."""
    import math
    s = 2 if dtype == "bf16" else 4
    total_d = total_k = total_stats = 0
    for shp in shapes:
        d = numel(shp)
        dbs = min(d, d_block_size)
        full = d // dbs
        k = full * math.ceil(dbs * k_init) + math.ceil((d - full * dbs) * k_init)
        total_d += d
        total_k += k
        total_stats += (d + q - 1) // q
    rows = sum(min(t, m) for t in range(first_step, first_step + n_steps)) / n_steps
    b = total_d * (s + 0.5 + 0.5 + 2 * s) + total_k * 4 * (1 + rows) + total_stats * 8
    if alpha > 0:
        b += total_d * 1.0  # the EF is read and written a second time
    return b / total_d


def cpu_baseline(workload, budget_s=12.0):
    """The C oracle on this host's cores, on a bounded sample of the workload."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import microadam_oracle as oracle
    oracle.build()
    shapes_fn, dtype, m, k_init, q, alpha, gstd = WORKLOADS[workload]
    shapes = shapes_fn()
    cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or min(os.cpu_count() or 1, 16)
    oracle.set_threads(cores)
    # sample: the first tensors of one repeating layer, up to ~200 M parameters
    sample, total = [], 0
    for shp in shapes[1:]:
        if total + numel(shp) > 210_000_000:
            break
        sample.append(shp)
        total += numel(shp)
    if not sample:
        sample, total = [shapes[0]], numel(shapes[0])
    rng = np.random.default_rng(0)

    def draw(n, std):
        x = rng.standard_normal(n, dtype=np.float32) * np.float32(std)
        return oracle.f32_to_bf16(x) if dtype == "bf16" else x

    params = [draw(numel(s), 0.02) for s in sample]
    opt = oracle.OracleMicroAdam(params, m, 1e-3, q, k_init, alpha)
    # two gradient sets in turn (the step overwrites the buffer it is given); the first m steps
    # fill the window and are not timed
    grad_sets = [[draw(numel(s), gstd) for s in sample] for _ in range(2)]
    for i in range(m):
        opt.step([g.copy() for g in grad_sets[i % 2]])
    steps, elapsed = 0, 0.0
    while steps < 1 or (elapsed < budget_s and steps < 40):
        grads = [g.copy() for g in grad_sets[steps % 2]]
        t0 = time.perf_counter()
        opt.step(grads)
        elapsed += time.perf_counter() - t0
        steps += 1
    return {"value": total * steps / elapsed, "unit": "params/s", "cores": cores, "kind": "port",
            "sample": f"{len(sample)} tensors ({total} params) of the {workload} list, "
                      f"{steps} timed steps after {m} to fill the window, "
                      f"C oracle with OpenMP"}


def route_label(opt, params):
    """Which route the optimizer takes for the tensors of the list, e.g. "fused" or
    "spanning" when all go one way, else counts per route."""
    names = {0: "op-by-op", 1: "fused", 2: "spanning", 3: "fused-densified"}
    counts = {}
    for p in params:
        r = opt._fusable(p, opt.state[p]) if opt.use_fused else 0
        counts[names[r]] = counts.get(names[r], 0) + 1
    return next(iter(counts)) if len(counts) == 1 else counts


def bench_sparse_window(args):
    """Sparse M-FAC's two kernels over the shared window layout at a ResNet-50-sized vector:
    a step is SP (scalar products of the m rows with a dense vector) followed by out.zero_() and
    LCG (linear combination of the rows), as in sparse_core_mfac_w_ef.py:185-226."""
    import math
    import torch
    import ista_daslab_cuda_sparse_mfac as smf
    from ista_daslab_optimizers import _hip

    d, dbs, m, k_init = 25_557_032, 20480, 1024, 0.01
    dev = torch.device("cuda:0")
    kb = math.ceil(dbs * k_init)
    tail = d - (d // dbs) * dbs
    k_few = math.ceil(tail * k_init) if tail else 0
    k = (d // dbs) * kb + k_few
    gen = torch.Generator(device=dev).manual_seed(0)
    I = torch.zeros(m, k, dtype=torch.int16, device=dev)
    V = torch.zeros(m, k, dtype=torch.bfloat16, device=dev)
    for r in range(m):  # rows as the optimizer makes them: block top-k of a dense vector
        x = torch.randn(d, generator=gen, device=dev).to(torch.bfloat16)
        _hip.check(_hip.lib.ma_block_topk(d, dbs, kb, k_few, _hip.dev_ptr(x), _hip.dev_ptr(I[r]),
                                          _hip.dev_ptr(V[r]), 0, _hip.MA_BF16, _hip.stream_ptr()),
                   "block_topk")
    g = torch.randn(d, generator=gen, device=dev).to(torch.bfloat16)
    coef = torch.randn(m, generator=gen, device=dev)
    dots = torch.zeros(m, dtype=torch.float32, device=dev)
    out = torch.zeros(d, dtype=torch.bfloat16, device=dev)
    warmup = 3 if args.warmup is None else args.warmup

    def one_step(events=None):
        dots.zero_()
        if events:
            events[0].record()
        smf.SP(0, 0, 23, d, m, k, dbs, kb, g, I, V, dots, 1)
        if events:
            events[1].record()
        out.zero_()
        if events:
            events[2].record()
        smf.LCG(0, 0, 51, d, m, k, dbs, kb, coef, I, V, out, 1)
        if events:
            events[3].record()

    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        one_step(ev[i])
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    sp_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    lcg_ms = sum(e[2].elapsed_time(e[3]) for e in ev) / args.steps
    window_bytes = m * k * 4
    sp_bytes = window_bytes + 2 * d + 4 * m        # window, g, out
    lcg_bytes = window_bytes + 4 * d + 4 * m       # window, out read and written, coefficients
    achieved = (sp_bytes + lcg_bytes) / ((sp_ms + lcg_ms) * 1e-3) / 1e9
    res = {
        "metric": "Sparse M-FAC window kernels, SP + LCG (params/s)",
        "value": d / (ms_per_step * 1e-3), "unit": "params/s", "n_gpus": 1, "steps": args.steps,
        "warmup": warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": args.workload, "storage": "bf16", "params": d, "m": m,
                   "k_init": k_init, "d_block_size": dbs, "k": k},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "sp_ms": sp_ms, "sp_gbs": sp_bytes / (sp_ms * 1e-3) / 1e9,
                     "lcg_ms": lcg_ms, "lcg_gbs": lcg_bytes / (lcg_ms * 1e-3) / 1e9},
    }
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import numpy as np
        import microadam_oracle as oracle
        rows = 32
        In = I[:rows].cpu().numpy()
        Vn = V[:rows].cpu().view(torch.int16).numpy().view(np.uint16)
        gn = g.cpu().view(torch.int16).numpy().view(np.uint16)
        t0 = time.perf_counter()
        oracle.sparse_scalar_products(d, rows, k, dbs, kb, gn, In, Vn, np.zeros(rows))
        oracle.sparse_linear_combination(d, rows, k, dbs, kb, coef[:rows].cpu().numpy(), In, Vn,
                                         np.zeros(d, dtype=np.uint16))
        cpu_s = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": d / (cpu_s * m / rows), "unit": "params/s", "cores": 1,
                               "kind": "port",
                               "sample": f"{rows} of the {m} window rows, time scaled by {m // rows}"}
    print(json.dumps(res))


class LaunchEvents:
    """Events on the launch stream right before and after every call of a step entry point of
    the library (each call enqueues all launches of its tensors and returns): the device time of
    a step is the time between them, added over the step's calls.  Events around step() as a
    whole also count the host's work of a step whenever the stream is empty, which is the case
    for the first steps after the synchronisation that starts the timed region."""
    ENTRY_POINTS = ("ma_fused_step", "ma_fused_step_densified", "ma_fused_step_quant_err",
                    "ma_spanning_step", "ma_logged_step")

    def __init__(self):
        import torch
        from ista_daslab_optimizers import _hip
        self.lib, self.steps, self.saved = _hip.lib, [], {}
        for name in self.ENTRY_POINTS:
            fn = getattr(self.lib, name)
            self.saved[name] = fn

            def timed(*a, _fn=fn):
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                e0.record()
                rc = _fn(*a)
                e1.record()
                self.steps[-1].append((e0, e1))
                return rc
            setattr(self.lib, name, timed)

    def begin_step(self):
        self.steps.append([])

    def restore(self):
        for name, fn in self.saved.items():
            setattr(self.lib, name, fn)

    def per_step_ms(self):
        return [sum(a.elapsed_time(b) for a, b in step) for step in self.steps]


def calibration(args):
    """Known-size streaming kernels on this device: the rate it sustains for reads, writes, a
    copy, the step's 2:1 read:write mix and the step's three large streams, with the step's own
    access shape (ma_stream_probe) and with stock torch kernels.  Prints one JSON line; the
    same kernels are what the FETCH_SIZE / WRITE_SIZE counters are scaled against."""
    import ctypes
    import torch
    from ista_daslab_optimizers import _hip
    dev = torch.device("cuda:0")
    nbytes = (args.calibration_gib << 30) // 40960 * 40960
    a = torch.empty(nbytes // 2, dtype=torch.bfloat16, device=dev).normal_()
    b = torch.empty(nbytes // 2, dtype=torch.bfloat16, device=dev).normal_()
    c = torch.empty(nbytes // 2, dtype=torch.bfloat16, device=dev)
    e = torch.zeros(nbytes // 4, dtype=torch.uint8, device=dev)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    reps = max(3, args.steps)

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
              for _ in range(reps)]
        for e0, e1 in ev:
            e0.record()
            fn()
            e1.record()
        torch.cuda.synchronize()
        ms = sorted(x.elapsed_time(y) for x, y in ev)
        return ms[len(ms) // 2]

    def probe(mode, nt, wgs=0):
        def run():
            stream_probe()(mode, nt, nbytes, wgs, a.data_ptr(), b.data_ptr(), c.data_ptr(),
                           e.data_ptr(), sink.data_ptr(), _hip.stream_ptr())
        return run

    moved = {0: nbytes, 1: nbytes, 2: 2 * nbytes, 3: 3 * nbytes, 4: 3 * nbytes + nbytes // 2,
             5: 2 * nbytes}
    names = {0: "read", 1: "write", 2: "copy", 3: "update (2 reads : 1 write)",
             4: "step streams (g, p, EF read; p, EF written)",
             5: "write, then read the same 40 KiB back"}
    rows = []
    for mode in range(6):
        for nt in (1, 0):
            for wgs in (0, 256 * 3 * 4):
                ms = timed(probe(mode, nt, wgs))
                rows.append({"kernel": "ma_stream_probe", "what": names[mode], "nontemporal": bool(nt),
                             "workgroups": wgs or nbytes // 40960, "bytes": moved[mode], "ms": ms,
                             "GB/s": moved[mode] / ms / 1e6})
    rows.append({"kernel": "torch copy_", "what": names[2], "bytes": 2 * nbytes,
                 "ms": (ms := timed(lambda: c.copy_(a))), "GB/s": 2 * nbytes / ms / 1e6})
    rows.append({"kernel": "torch add(out=)", "what": "c = a + b (2 reads : 1 write)",
                 "bytes": 3 * nbytes, "ms": (ms := timed(lambda: torch.add(a, b, out=c))),
                 "GB/s": 3 * nbytes / ms / 1e6})
    rows.append({"kernel": "torch add_", "what": names[3], "bytes": 3 * nbytes,
                 "ms": (ms := timed(lambda: b.add_(a))), "GB/s": 3 * nbytes / ms / 1e6})
    rows.append({"kernel": "torch fill_", "what": names[1], "bytes": nbytes,
                 "ms": (ms := timed(lambda: c.fill_(1.0))), "GB/s": nbytes / ms / 1e6})
    rows.append({"kernel": "torch sum", "what": names[0], "bytes": nbytes,
                 "ms": (ms := timed(lambda: a.view(torch.int16).sum())),
                 "GB/s": nbytes / ms / 1e6})
    best = max(r["GB/s"] for r in rows if r["what"] == names[4])
    print(json.dumps({"calibration": rows, "bytes_per_array": nbytes, "reps": reps,
                      "peak_GB/s": HBM_PEAK_GBS, "step_streams_best_GB/s": best,
                      "step_streams_best_frac_of_peak": best / HBM_PEAK_GBS}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps; default m + 2, so that the window is full when timing starts")
    ap.add_argument("--workload", default="llama2-7b",
                    choices=sorted(WORKLOADS) + ["sparse-mfac-resnet50"])
    ap.add_argument("--grad-sets", type=int, default=None,
                    help="distinct resident gradient sets used in turn; default m + 2 (no gradient "
                         "recurs inside the window, as when gradients are redrawn every step) or as "
                         "many as fit in 60 %% of the device memory")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--op-by-op", action="store_true", help="time the unfused route instead")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain device copy of CAL_BYTES (ma_stream_probe, mode 2), the "
                         "known-size kernel the FETCH_SIZE / WRITE_SIZE counters are scaled against")
    ap.add_argument("--calibration", action="store_true",
                    help="time known-size streaming kernels instead of the optimizer step")
    ap.add_argument("--calibration-gib", type=int, default=4, help="bytes per array, GiB")
    ap.add_argument("--grad-scale-drift", type=float, default=0.0,
                    help="multiply the gradients of step i by (1 + drift)^i (set on the device "
                         "before the step, outside the timed kernels): with a drift well above the "
                         "1/32 margin of the hinted top-k selection its bound fails in every block "
                         "and the step pays the fallback selection")
    ap.add_argument("--storage", choices=["bf16", "f32"], default=None,
                    help="override the element type of parameters and gradients")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X: this build has no multi-GPU path, run with --gpus 1")

    if args.calibration:
        return calibration(args)
    if args.workload == "sparse-mfac-resnet50":
        return bench_sparse_window(args)

    import torch
    from ista_daslab_optimizers import MicroAdam

    shapes_fn, dtype, m, k_init, q, alpha, gstd = WORKLOADS[args.workload]
    if args.warmup is None:
        args.warmup = m + 2
    if args.storage is not None:
        dtype = args.storage
    shapes = shapes_fn()
    tdtype = torch.bfloat16 if dtype == "bf16" else torch.float32
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    params = []
    for shp in shapes:
        p = torch.empty(shp, dtype=tdtype, device=dev)
        p.normal_(0, 0.02)
        params.append(torch.nn.Parameter(p))
    n_params = sum(p.numel() for p in params)
    if args.grad_sets is None:
        esize = 2 if dtype == "bf16" else 4
        free = 0.6 * torch.cuda.get_device_properties(dev).total_memory - 3 * esize * n_params
        args.grad_sets = int(max(1, min(m + 2, free // (esize * n_params))))
    grad_sets = []
    for _ in range(max(1, args.grad_sets)):
        gs = []
        for shp in shapes:
            g = torch.empty(shp, dtype=tdtype, device=dev)
            g.normal_(0, gstd)
            gs.append(g)
        grad_sets.append(gs)

    opt = MicroAdam(params, m=m, lr=1e-3, quant_block_size=q, k_init=k_init, alpha=alpha,
                    betas=(0.9, 0.999), eps=1e-8, weight_decay=0)
    opt.use_fused = not args.op_by_op

    scale_of = {}

    def prepare(i):
        """--grad-scale-drift: the gradient set of step i brought to that step's level."""
        if args.grad_scale_drift:
            which = i % len(grad_sets)
            now = (1.0 + args.grad_scale_drift) ** i
            torch._foreach_mul_(grad_sets[which], now / scale_of.get(which, 1.0))
            scale_of[which] = now

    def one_step(i):
        gs = grad_sets[i % len(grad_sets)]
        for p, g in zip(params, gs):
            p.grad = g
        opt.step()

    for i in range(args.warmup):
        prepare(i)
        one_step(i)
    torch.cuda.synchronize()
    if args.copy_calibration:
        # one plain copy of known size (ma::stream_kernel<2, true>): reads CAL_BYTES, writes CAL_BYTES
        from ista_daslab_optimizers import _hip
        src = torch.empty(CAL_BYTES // 2, dtype=torch.bfloat16, device=dev).normal_()
        dst = torch.empty_like(src)
        sink = torch.zeros(1, dtype=torch.int32, device=dev)
        stream_probe()(2, 1, CAL_BYTES, 0, src.data_ptr(), None, dst.data_ptr(), None,
                       sink.data_ptr(), _hip.stream_ptr())
        torch.cuda.synchronize()
        del src, dst
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(args.steps)]
    calls = LaunchEvents()
    host = 0.0  # time the host spends inside step() (the kernels run behind it)
    t0 = time.perf_counter()
    for i in range(args.steps):
        prepare(args.warmup + i)  # (its kernels run between the events of two steps)
        ev[i][0].record()
        h0 = time.perf_counter()
        calls.begin_step()
        one_step(args.warmup + i)
        host += time.perf_counter() - h0
        ev[i][1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    calls.restore()
    span_series = [a.elapsed_time(b) for a, b in ev]  # in step order
    # the launches of a step, timed on their stream; the op-by-op route (one library call and a
    # few torch kernels per operation) has no step entry point to bracket: its steps are
    # timed from the events around step()
    dev_series = calls.per_step_ms() if all(calls.steps) else span_series
    dev_ms = sorted(dev_series)
    ms_per_step = wall * 1e3 / args.steps
    kernel_ms = sum(dev_ms) / len(dev_ms)

    traffic, traffic_source = (MEASURED_TRAFFIC.get((args.workload, args.op_by_op), (None, None))
                               if args.storage is None and not args.grad_scale_drift
                               else (None, None))
    bpp = algorithmic_bytes_per_param(shapes, dtype, m, k_init, q, alpha, opt.d_block_size,
                                      args.warmup + 1, args.steps)
    achieved = bpp * n_params / (kernel_ms * 1e-3) / 1e9
    out = {
        "metric": "MicroAdam step throughput (params/s) at the Llama-2-7B shape"
                  if args.workload == "llama2-7b" else f"MicroAdam step throughput ({args.workload})",
        "value": n_params / (ms_per_step * 1e-3),
        "unit": "params/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "host_ms_per_step": host * 1e3 / args.steps,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",  # arithmetic type; storage type of p and g is config.storage
        "data": "synthetic",
        "config": {"workload": args.workload, "storage": dtype, "params": n_params,
                   "grad_sets": args.grad_sets,
                   "tensors": len(shapes), "m": m,
                   "k_init": k_init, "quant_block_size": q, "alpha": alpha,
                   "d_block_size": opt.d_block_size, "grad_scale_drift": args.grad_scale_drift,
                   "route": route_label(opt, params)},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     # counters cannot be read from inside this run: the figure is the one the
                     # same workload measured under rocprofv3 --pmc, kept in the file named
                     "traffic": traffic, "traffic_source": traffic_source,
                     # achieved and traffic are both per step (at 7B: 2 launches of the block
                     # kernel): algorithmic bytes of a step / device time of a step
                     "per": "step", "algorithmic_bytes": bpp * n_params,
                     "bytes_per_param": bpp, "device_ms_per_step": kernel_ms,
                     "device_ms_min": dev_ms[0], "device_ms_median": dev_ms[len(dev_ms) // 2],
                     "device_ms_series": [round(x, 3) for x in dev_series],
                     # events around the whole of step(): on top of the launches, the host's
                     # share of a step whenever the stream has run dry (the first timed steps)
                     "step_events_ms_per_step": sum(span_series) / len(span_series)},
    }
    if not args.no_cpu_baseline:
        del grad_sets
        out["cpu_baseline"] = cpu_baseline(args.workload)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
