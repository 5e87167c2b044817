"""The C-ABI library loads and exports every symbol include/microadam_hip.h declares; the host
helpers mirror the reference's; without a GPU the optimizer refuses to run instead of falling
back to anything.  No compute calls here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "microadam_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ma_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from ista_daslab_optimizers import _hip
    names = _declared()
    assert len(names) >= 13
    lib = ctypes.CDLL(_hip.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert set(_hip.EXPORTS) == set(names)
    assert _hip.lib.ma_get_max_floats_for_shared_memory_per_thread_block() == 40960
    assert "window" in _hip.error_string(-3)


def test_struct_layouts_match_header():
    from ista_daslab_optimizers import _hip
    # struct ma_tensor: 7 pointers, 2 int64, 2 double, 2 int32; struct ma_hyper: see header
    assert ctypes.sizeof(_hip.MaTensor) == 7 * 8 + 2 * 8 + 2 * 8 + 2 * 4 + 8 + 8
    assert ctypes.sizeof(_hip.MaHyper) == 8 + 4 + 4 + 8 + 8 + 4 * 8
    assert _hip.MaTensor.lr.offset == 72 and _hip.MaTensor.index.offset == 88
    assert _hip.MaTensor.quant_err.offset == 96 and _hip.MaTensor.row_cuts.offset == 104


def test_host_helpers_mirror_reference():
    from ista_daslab_optimizers.tools import CopyDirection, block_split
    assert (CopyDirection.k2d.value, CopyDirection.d2k.value) == (0, 1)
    assert block_split(5, 10) == (1, 5)
    assert block_split(16777216, 20480) == (819, 16773120)


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU behaviour")
def test_no_gpu_is_an_error_not_a_fallback():
    from ista_daslab_optimizers import MicroAdam
    p = torch.nn.Parameter(torch.zeros(128))
    with pytest.raises(RuntimeError):
        MicroAdam([p], m=3, lr=1e-3, quant_block_size=64)


def test_fused_step_check_rejects_bad_layouts():
    """Host-only validation of ma_fused_step's conditions (nothing is launched)."""
    from ista_daslab_optimizers import _hip
    t = _hip.MaTensor()
    for f in ("p", "g", "error", "min_vals", "max_vals", "I", "V"):
        setattr(t, f, 0x10000)
    t.d, t.k, t.lr, t.weight_decay, t.index = 20480 * 2 + 4096, 205 * 2 + 41, 1e-3, 0.0, 0
    h = _hip.MaHyper(1, 10, _hip.MA_BF16, 64, 20480, 0.01, 0.9, 0.999, 1e-8)
    chk = lambda: _hip.lib.ma_fused_step_check(ctypes.byref(t), ctypes.byref(h))
    assert chk() == 0
    t.k += 1
    assert chk() == -4  # geometry
    t.k -= 1
    h.quant_block_size = 100000
    assert chk() == _hip.MA_ERR_NOT_FUSABLE
    h.quant_block_size = 64
    t.g = 0x10002
    assert chk() == _hip.MA_ERR_NOT_FUSABLE
    t.g = 0x10000
    h.m = 65
    assert chk() == -3


def test_step_checks_refuse_what_does_not_fit_in_lds():
    """The admission checks lay out the LDS of the launch the tensor would get: a selection of
    70 % of a 20480-element fp32 block needs more than the 160 KB a workgroup can have, so the
    tensor is refused (and the optimizer then steps it op by op) instead of failing at launch."""
    from ista_daslab_optimizers import _hip
    import math
    d = 20480 * 2
    t = _hip.MaTensor()
    for f in ("p", "g", "error", "min_vals", "max_vals", "I", "V"):
        setattr(t, f, 0x10000)
    t.d, t.lr, t.weight_decay, t.index = d, 1e-3, 0.0, 0
    for k_init, want in ((0.01, 0), (0.7, _hip.MA_ERR_LDS)):
        t.k = 2 * int(math.ceil(20480 * k_init))
        h = _hip.MaHyper(1, 10, _hip.MA_F32, 64, 20480, k_init, 0.9, 0.999, 1e-8)
        assert _hip.lib.ma_fused_step_check(ctypes.byref(t), ctypes.byref(h)) == want, k_init
        h.quant_block_size = 40960
        assert _hip.lib.ma_spanning_step_check(ctypes.byref(t), ctypes.byref(h), 0.5) == want, k_init


def test_row_cuts_query():
    """Host-only: which tensors ma_fused_step keeps a cache of row cuts for, and its size."""
    from ista_daslab_optimizers import _hip
    import math
    t = _hip.MaTensor()
    for f in ("p", "g", "error", "min_vals", "max_vals", "I", "V"):
        setattr(t, f, 0x10000)
    t.lr, t.weight_decay, t.index = 1e-3, 0.0, 0

    def words(d, m, k_init, dtype=_hip.MA_BF16):
        dbs = min(d, 20480)
        t.d = d
        t.k = d // dbs * int(math.ceil(dbs * k_init)) + int(math.ceil(d % dbs * k_init))
        h = _hip.MaHyper(1, m, dtype, 64, 20480, k_init, 0.9, 0.999, 1e-8)
        return _hip.lib.ma_fused_step_row_cuts(ctypes.byref(t), ctypes.byref(h))

    # 20 rows of 1024 entries per block: two launches, 41 cuts for each of the 3 blocks
    assert words(20480 * 2 + 4096, 20, 0.05) == 3 * 41
    assert words(20480 * 2, 20, 0.05) == 2 * 41
    # the window of the 7B configuration fits the one-pass stage
    assert words(20480 * 2 + 4096, 10, 0.01) == 0
    # two launches, but rows of at most 512 entries are not listed by coordinate
    assert words(20480 * 2, 20, 0.01) == 0
    # a tensor shorter than a top-k block: one block, ceil(d / 512) + 1 cuts
    assert words(16384, 20, 0.05) == 33
    assert _hip.lib.ma_fused_step_row_cuts(None, None) == _hip.MA_ERR_ARG


def test_logged_step_argument_checks():
    """Host-only: the size of the per-block buffer a logging step needs, and the refusals that
    come before any launch."""
    from ista_daslab_optimizers import _hip
    t = _hip.MaTensor()
    for f in ("p", "g", "error", "min_vals", "max_vals", "I", "V"):
        setattr(t, f, 0x10000)
    t.d, t.k, t.lr, t.weight_decay, t.index = 20480 * 2 + 4096, 205 * 2 + 41, 1e-3, 0.0, 0
    h = _hip.MaHyper(1, 10, _hip.MA_BF16, 64, 20480, 0.01, 0.9, 0.999, 1e-8)
    assert _hip.lib.ma_logged_step_partials(ctypes.byref(t), 1, ctypes.byref(h)) == 3 * 8
    assert _hip.lib.ma_logged_step_partials(None, 1, ctypes.byref(h)) == -1
    call = lambda route, partials, n, sums: _hip.lib.ma_logged_step(
        route, ctypes.byref(t), 1, ctypes.byref(h), 0.0, None, 0, partials, n, sums, None)
    assert call(_hip.MA_ROUTE_FUSED, 0x10000, 24, None) == _hip.MA_ERR_ARG        # no sums
    assert call(_hip.MA_ROUTE_FUSED, 0x10000, 23, 0x10000) == _hip.MA_ERR_ARG     # buffer too short
    assert call(_hip.MA_ROUTE_FUSED, None, 24, 0x10000) == _hip.MA_ERR_ARG
    assert call(7, 0x10000, 24, 0x10000) == _hip.MA_ERR_ARG                       # unknown route
    assert call(_hip.MA_ROUTE_DENSIFIED, 0x10000, 24, 0x10000) == _hip.MA_ERR_NOT_FUSABLE  # alpha 0


def test_spanning_step_check_and_workspace():
    """Host-only validation of ma_spanning_step's conditions and its workspace size."""
    from ista_daslab_optimizers import _hip
    t = _hip.MaTensor()
    for f in ("p", "g", "error", "min_vals", "max_vals", "I", "V"):
        setattr(t, f, 0x10000)
    t.d, t.k, t.lr, t.weight_decay, t.index = 20480 * 2 + 4096, 205 * 2 + 41, 1e-3, 0.0, 0
    h = _hip.MaHyper(1, 10, _hip.MA_BF16, 100000, 20480, 0.01, 0.9, 0.999, 1e-8)
    chk = lambda a: _hip.lib.ma_spanning_step_check(ctypes.byref(t), ctypes.byref(h), a)
    assert chk(0.5) == 0
    assert chk(0.0) == 0
    assert chk(-2.0) == _hip.MA_ERR_NOT_FUSABLE
    assert chk(1.0) == _hip.MA_ERR_NOT_FUSABLE      # micro_adam.py:18 asks for alpha < 1
    h.quant_block_size = 100001                     # not a multiple of 8
    assert chk(0.5) == _hip.MA_ERR_NOT_FUSABLE
    h.quant_block_size = 64                         # shorter than the top-k block
    assert chk(0.5) == _hip.MA_ERR_NOT_FUSABLE
    h.quant_block_size = 20480 * 100                # covers more top-k blocks than one wave reads
    assert chk(0.5) == _hip.MA_ERR_NOT_FUSABLE
    h.quant_block_size = 100000
    arr = (_hip.MaTensor * 2)(t, t)
    assert _hip.lib.ma_spanning_step_workspace(arr, 2, ctypes.byref(h)) == 2 * 3 * 32
    # too small a workspace is refused before anything is launched
    rc = _hip.lib.ma_spanning_step(arr, 2, ctypes.byref(h), 0.5, 0x10000, 16, None)
    assert rc == -1  # MA_ERR_ARG
