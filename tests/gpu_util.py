"""Helpers shared by the GPU parity tests: moving data between torch (GPU), numpy (oracle)."""
import numpy as np
import torch


def to_np(t):
    """GPU/CPU torch tensor -> numpy array in the oracle's convention (bf16 as uint16 bits)."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def to_torch(a, device="cuda"):
    """numpy array in the oracle's convention -> torch tensor (uint16 becomes bf16)."""
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).to(device)
    return torch.from_numpy(a.copy()).to(device)


def rand_vec(gen, n, dtype, scale=1.0):
    """Seeded CPU draw, returned as a CPU torch tensor of `dtype`."""
    return (torch.randn(n, generator=gen) * scale).to(dtype)


def state_snapshot(st):
    return {k: to_np(st[k]) for k in ("I", "V", "error", "min_vals", "max_vals")}


def assert_state_equal(gst, ost, ctx=""):
    """Bit-exact comparison of a GPU optimizer state with the oracle's.  The window is compared
    as index sets with their values: entries of a block row are sorted by index first, since
    their order inside the block is unspecified (torch.topk(sorted=False) in the reference)."""
    import microadam_oracle as oracle
    snap = state_snapshot(gst)
    assert gst["index"] == ost["index"], ctx
    km = ost["k_block_size_many"]
    snap["I"], snap["V"] = oracle.canonical_window(snap["I"], snap["V"], km)
    ost = dict(ost)
    ost["I"], ost["V"] = oracle.canonical_window(ost["I"], ost["V"], km)
    for key in ("I", "V", "error", "min_vals", "max_vals"):
        a, b = snap[key], np.asarray(ost[key]).reshape(snap[key].shape)
        if not np.array_equal(a, b):
            bad = np.nonzero(a.reshape(-1) != b.reshape(-1))[0]
            raise AssertionError(f"{ctx}: state[{key!r}] differs at {bad.size} of {a.size} "
                                 f"entries, first at {bad[:5]}: gpu {a.reshape(-1)[bad[:5]]} "
                                 f"oracle {b.reshape(-1)[bad[:5]]}")
