"""MicroAdam on MI355X.

Same class name, constructor, attributes and per-parameter state as the optimizer of
ista_daslab_optimizers/micro_adam/micro_adam.py (constructor :14, state :61-94); the step itself
is carried out by gfx950 HIP kernels of libmicroadam_hip.so.  Every tensor of a step takes one
of four routes, all of which compute micro_adam.py:146-328:

  fused            ma_fused_step            alpha == 0, quantisation blocks inside the top-k blocks
  fused, densified ma_fused_step_densified  0 < alpha < 1, same layout
  spanning         ma_spanning_step         0 <= alpha < 1, quantisation blocks at least as long
                                            as the top-k blocks
  op by op         one kernel per call of the reference's sequence: everything else
                   (alpha == -2, other quantisation block sizes, unaligned or strided tensors)

The fused routes take all their tensors in one library call per element type; what the call
needs per tensor (seven device addresses, sizes, lr, weight decay, ring position) lives in a
table that is built once and refreshed in place.  There is no CPU or pure-PyTorch route: a
missing library, a missing GPU or a CPU tensor raises.
"""
import ctypes
import math
import time

import numpy as np
import torch
import torch.distributed as dist

import ista_daslab_cuda_micro_adam as _ext_quant
import ista_daslab_cuda_tools as _ext_tools

from .. import _hip
from ..tools import block_split, get_first_device, get_gpu_mem_usage

try:  # logging is optional here; the reference imports wandb unconditionally (micro_adam.py:5)
    import wandb
except Exception:  # pragma: no cover
    wandb = None

OP_BY_OP, FUSED, SPANNING, FUSED_DENSIFIED, FUSED_QUANT_ERR = 0, 1, 2, 3, 4
_LOGGED_ROUTE = {FUSED: _hip.MA_ROUTE_FUSED, FUSED_DENSIFIED: _hip.MA_ROUTE_DENSIFIED,
                 SPANNING: _hip.MA_ROUTE_SPANNING, FUSED_QUANT_ERR: _hip.MA_ROUTE_QUANT_ERR}

# state tensors whose element type the kernels depend on (micro_adam.py:86-94)
_TYPED_STATE = (('I', torch.int16), ('V', torch.bfloat16), ('error', torch.uint8),
                ('min_vals', torch.bfloat16), ('max_vals', torch.bfloat16))

_TENSOR_RECORD = np.dtype([(name, np.uint64 if ctype is ctypes.c_void_p else
                            {ctypes.c_int64: np.int64, ctypes.c_double: np.float64,
                             ctypes.c_int32: np.int32}[ctype])
                           for name, ctype in _hip.MaTensor._fields_], align=True)
assert _TENSOR_RECORD.itemsize == ctypes.sizeof(_hip.MaTensor)


def _distributed():
    return dist.is_available() and dist.is_initialized()


class _Table:
    """The ma_tensor records of one fused route and element type, as a ctypes array for the
    library and a numpy view of the same memory for refreshing whole columns at once."""

    def __init__(self, entries):
        self.entries = entries
        self.records = (_hip.MaTensor * len(entries))()
        self.view = np.frombuffer(self.records, dtype=_TENSOR_RECORD)
        for name in ('error', 'min_vals', 'max_vals', 'I', 'V'):
            self.view[name] = [e.st[name].data_ptr() for e in entries]
        self.view['quant_err'] = [e.st['quant_err'].data_ptr() if 'quant_err' in e.st else 0
                                  for e in entries]
        self.view['row_cuts'] = [0 if e.cuts is None else e.cuts.data_ptr() for e in entries]
        self.view['d'] = [e.st['d'] for e in entries]
        self.view['k'] = [e.st['k'] for e in entries]

    def refresh(self):
        es = self.entries
        self.view['p'] = [e.p_addr for e in es]
        self.view['g'] = [e.g_addr for e in es]
        self.view['lr'] = [e.lr for e in es]
        self.view['weight_decay'] = [e.wd for e in es]
        self.view['index'] = [e.st['index'] for e in es]


class _Entry:
    """What the step knows about one parameter between steps."""
    __slots__ = ('p', 'st', 'route', 'lr', 'wd', 'p_addr', 'g_addr', 'cuts')

    def __init__(self, p, st, route):
        self.p, self.st, self.route = p, st, route
        self.lr = self.wd = 0.0
        self.p_addr = self.g_addr = 0  # device addresses of p and p.grad in the current step
        # ma_fused_step's cache of where each window row crosses the multiples of 512
        # coordinates (include/microadam_hip.h, ma_fused_step_row_cuts): not part of the state,
        # rebuilt row by row after a reload; None when the tensor's step has no use for it
        self.cuts = None

    def forget_row_cuts(self, row):
        """Row `row` of the window is being written by something else than ma_fused_step."""
        if self.cuts is not None:
            self.cuts[row].fill_(-1)


class MicroAdam(torch.optim.Optimizer):
    def __init__(self, params, m, lr, quant_block_size, k_init=0.01, alpha=0, betas=(0.9, 0.999),
                 weight_decay=0, eps=1e-8):
        super().__init__(params, dict(lr=lr, weight_decay=weight_decay, eps=eps, alpha=alpha))
        assert (0 <= alpha < 1) or alpha == -2, 'Alpha must be in the [0, 1) interval or -2'

        self.m, self.lr, self.k_init, self.alpha = m, lr, k_init, alpha
        self.quant_block_size = int(quant_block_size)
        self.weight_decay, self.eps = weight_decay, eps
        self.beta1, self.beta2 = betas
        self.densify_update_using_ef = alpha > 0
        self.densify_update_using_quant_error = alpha == -2

        every = [p for group in self.param_groups for p in group['params']]
        self.model_size = sum(p.numel() for p in every)
        self.steps = 0
        self.log_interval = 100
        self.device = get_first_device()
        self._is_state_initialized = False

        # launch geometry the reference asks its extension for (micro_adam.py:39-44)
        self.shared_memory_carveout = 100
        share = int(100 / self.shared_memory_carveout)
        self.blocks = _ext_tools.get_sm_count() * share
        self.threads = 512
        self.max_floats = _ext_tools.get_max_floats_for_shared_memory_per_thread_block()
        self.d_block_size = self.max_floats // 2 // share

        # how many tensors of each size there are: overall, and per rank once the first step has
        # seen which of them this rank holds (micro_adam.py:46-57, :107-114)
        ranks = dist.get_world_size() if _distributed() else 1
        self.fsdp_dict_size_count = [{} for _ in range(ranks)]
        self.dict_size_count = {}
        for p in every:
            self.dict_size_count[p.numel()] = 1 + self.dict_size_count.get(p.numel(), 0)

        # not in the reference: route selection and the tables of the fused routes
        self.use_fused = True
        self._entries = {}     # parameter -> _Entry (holds the parameter, so ids are not reused)
        self._tables = {}      # (route, dtype) -> _Table
        self._walk = None      # per parameter group: (group, its parameter list, their entries)
        self._workspace = None  # device scratch of the spanning route, grown on demand
        self._partials = None   # per-block sums of a logging step, grown on demand

    # ------------------------------------------------------------------ state (micro_adam.py:61-94)
    def _initialize_parameter_state(self, p, lr, wd):
        d = p.numel()
        st = self.state[p]
        rank = dist.get_rank() if _distributed() else 0
        if self.densify_update_using_quant_error:
            st['quant_err'] = torch.zeros_like(p)

        same_size = self.fsdp_dict_size_count[rank].get(d, 1)
        st['blocks'] = max(1, int(math.floor(self.blocks * d * same_size / self.model_size)))
        st['lr'], st['weight_decay'], st['d'] = lr, wd, d

        # top-k blocks: full ones of d_block_size and a shorter last one starting at d_index_topk
        dbs = min(d, self.d_block_size)
        full, tail_start = block_split(d, dbs)
        per_full = int(math.ceil(dbs * self.k_init))
        per_tail = int(math.ceil((d - tail_start) * self.k_init))
        st['d_block_size'] = dbs
        st['topk_full_blocks_count'], st['d_index_topk'] = full, tail_start
        st['k_block_size_many'], st['k_block_size_few'] = per_full, per_tail
        st['k_index'] = full * per_full
        st['k'] = full * per_full + per_tail

        # the window: m rows of k (block-relative index, value) pairs, written round robin
        st['index'] = 0
        st['I'] = torch.zeros(self.m, st['k'], dtype=torch.int16, device=p.device)
        st['V'] = torch.zeros(self.m, st['k'], dtype=torch.bfloat16, device=p.device)

        # 4-bit error feedback with one (min, max) pair per quantisation block
        q_full, q_tail_start = block_split(d, self.quant_block_size)
        st['quant_full_blocks_count'], st['d_index_quant'] = q_full, q_tail_start
        st['error'] = torch.zeros(int(math.ceil(d / 2)), dtype=torch.uint8, device=p.device)
        st['min_vals'] = torch.zeros(q_full + 1, dtype=torch.bfloat16, device=p.device)
        st['max_vals'] = torch.zeros(q_full + 1, dtype=torch.bfloat16, device=p.device)

    @staticmethod
    def _check_param(p):
        if not p.is_cuda:
            raise RuntimeError(f"MicroAdam runs on the GPU only; got a parameter on {p.device}")
        if p.dtype not in (torch.float32, torch.bfloat16):
            raise TypeError(f"MicroAdam takes float32 or bfloat16 parameters, got {p.dtype}")

    def _repair_state(self, st):
        """Frameworks that reload or re-type optimizer state cast every state tensor to the
        parameter's dtype (the reference repairs st['I'] for this reason, micro_adam.py:175-178);
        the kernels need the declared types back.  True if a tensor was replaced."""
        replaced = False
        for key, dtype in _TYPED_STATE:
            if st[key].dtype != dtype:
                st[key] = st[key].to(dtype)
                replaced = True
        return replaced

    def _entry(self, p, lr, wd):
        """State of p (created at first touch, micro_adam.py:158-160) and its cached route."""
        st = self.state[p]
        if len(st) == 0:
            self._check_param(p)
            self._initialize_parameter_state(p, lr, wd)
        repaired = self._repair_state(st)
        if self.densify_update_using_quant_error and 'quant_err' not in st:
            st['quant_err'] = torch.zeros_like(p)  # state loaded from a run with another alpha
            repaired = True
        e = self._entries.get(p)
        if e is None or e.st is not st or repaired:
            e = self._entries[p] = _Entry(p, st, self._static_route(p, st))
            if e.route == FUSED:
                probe, h = self._probe(p, st)
                words = _hip.lib.ma_fused_step_row_cuts(ctypes.byref(probe), ctypes.byref(h))
                if words > 0:
                    e.cuts = torch.full((self.m, words), -1, dtype=torch.int16, device=p.device)
            self._tables.clear()
        return e

    # ------------------------------------------------------------------ routes
    def _static_route(self, p, st):
        """The route the tensor's sizes and the hyper-parameters admit (the conditions of
        ma_fused_step / ma_spanning_step in include/microadam_hip.h), checked by the library
        itself where it offers the check; what depends on this step's buffers is _fusable's."""
        if not (0 <= self.alpha < 1 or self.alpha == -2) or self.m > _hip.MA_MAX_WINDOW:
            return OP_BY_OP
        # state made for another top-k block size (a checkpoint from other hardware) runs op by
        # op from its stored geometry; the fused kernels derive theirs from self.d_block_size
        d, dbs = st['d'], st['d_block_size']
        expect_k = (int(math.ceil(dbs * self.k_init)) * (d // dbs)
                    + int(math.ceil((d - d // dbs * dbs) * self.k_init)))
        if dbs != min(d, self.d_block_size) or st['k'] != expect_k:
            return OP_BY_OP
        probe, h = self._probe(p, st)
        if _hip.lib.ma_fused_step_check(ctypes.byref(probe), ctypes.byref(h)) == 0:
            if self.alpha == -2:
                return FUSED_QUANT_ERR
            if self.alpha == 0:
                return FUSED
            return FUSED_DENSIFIED
        if self.alpha == -2:
            return OP_BY_OP
        if _hip.lib.ma_spanning_step_check(ctypes.byref(probe), ctypes.byref(h),
                                           float(self.alpha)) == 0:
            return SPANNING
        return OP_BY_OP

    def _probe(self, p, st):
        """A record of p's state (with stand-ins for the buffers of a step) and the
        hyper-parameters, for the library's admission and size queries."""
        probe = _hip.MaTensor()
        for name in ('p', 'g'):
            setattr(probe, name, 256)  # stands for any 16-byte aligned address
        for name, _ in _TYPED_STATE:
            setattr(probe, name, st[name].data_ptr())
        probe.d, probe.k, probe.index = st['d'], st['k'], 0
        return probe, self._hyper(p.dtype, max(self.steps, 1))

    def _fusable(self, p, st):
        """Route p takes in a step with its current gradient: 0 op by op, 1 fused, 2 spanning,
        3 fused densified, 4 fused with alpha == -2."""
        g = p.grad
        if g.dtype != p.dtype or not p.is_contiguous() or not g.is_contiguous():
            return OP_BY_OP
        if (p.data_ptr() | g.data_ptr()) & 15:
            return OP_BY_OP
        e = self._entries.get(p)
        if e is None or e.st is not st:
            return self._static_route(p, st)
        return e.route

    def _hyper(self, dtype, t):
        return _hip.MaHyper(t, self.m, _hip.MA_BF16 if dtype == torch.bfloat16 else _hip.MA_F32,
                            self.quant_block_size, self.d_block_size, self.k_init, self.beta1,
                            self.beta2, self.eps)

    # ------------------------------------------------------------------ step (micro_adam.py:96-144)
    @torch.no_grad()
    def step(self, closure=None):
        self.steps += 1
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        if self.steps == 1:
            mine = self.fsdp_dict_size_count[dist.get_rank() if _distributed() else 0]
            for group in self.param_groups:
                for p in group['params']:
                    if p is not None and p.numel() > 0:
                        mine[p.numel()] = 1 + mine.get(p.numel(), 0)

        started = time.time()
        logging_step = self._logging_active() and self.steps % self.log_interval == 0
        totals = dict(norm_qe=0, norm_g=0, norm_u=0, norm_e=0, sparsity_u=0, sparsity_qe=0)
        batches = {}  # (route, dtype) -> entries, in parameter order
        fused_allowed = self.use_fused
        for group, plist, entries in self._groups():
            lr = group['lr']
            wd = group.get('weight_decay', self.weight_decay)
            for i, p in enumerate(plist):
                g = None if p is None else p.grad
                if g is None:
                    continue
                e = entries[i]
                if e is None or e.st['I'].dtype is not torch.int16:
                    e = entries[i] = self._entry(p, lr, wd)
                # what this step's buffers admit: same element type, dense, 16-byte aligned
                route = OP_BY_OP
                if (fused_allowed and e.route and g.dtype is p.dtype and g.is_contiguous()
                        and p.is_contiguous()):
                    e.p_addr, e.g_addr = p.data_ptr(), g.data_ptr()
                    if not (e.p_addr | e.g_addr) & 15:
                        route = e.route
                if route == OP_BY_OP:
                    for key, value in self.update_step(p, lr, wd, logging_step).items():
                        totals[key] += value
                    continue
                e.lr, e.wd = lr, wd
                batch = batches.get((route, p.dtype))
                if batch is None:
                    batch = batches[(route, p.dtype)] = []
                batch.append(e)

        sums = None  # the fused routes' shares of the logged sums, formed by their kernels
        for (route, dtype), entries in batches.items():
            if logging_step and sums is None:
                sums = torch.zeros(8, dtype=torch.float64, device=entries[0].p.device)
            self._fused_step(route, dtype, entries, sums)
        if sums is not None:
            for key, value in zip(('norm_qe', 'norm_g', 'norm_u', 'norm_e', 'sparsity_u',
                                   'sparsity_qe'), sums.tolist()):
                totals[key] += value

        if logging_step:
            self._log(totals['norm_qe'], totals['norm_g'], totals['norm_u'], totals['norm_e'],
                      totals['sparsity_u'], totals['sparsity_qe'], time.time() - started)
        return loss

    def _groups(self):
        """The parameter groups with the cached entries of their parameters, rebuilt when a
        group was added or a group's parameter list replaced or resized."""
        walk = self._walk
        groups = self.param_groups
        if walk is None or len(walk) != len(groups) or any(
                w[0] is not g or w[1] is not g['params'] or len(w[2]) != len(w[1])
                for w, g in zip(walk, groups)):
            walk = self._walk = [(g, g['params'], [self._entries.get(p) for p in g['params']])
                                 for g in groups]
        return walk

    # ------------------------------------------------------------------ fused routes
    def _fused_step(self, route, dtype, entries, sums=None):
        """One library call for the tensors of one route and element type.  sums: None, or the
        8 float64 on the device that a logging step's kernels add their sums to
        (micro_adam.py:155-156, :271-272, :306-308, :320-324)."""
        table = self._tables.get((route, dtype))
        if table is None or len(table.entries) != len(entries) or any(
                a is not b for a, b in zip(table.entries, entries)):
            table = self._tables[(route, dtype)] = _Table(list(entries))
        table.refresh()
        n, h, stream = len(entries), self._hyper(dtype, self.steps), _hip.stream_ptr()
        device = entries[0].p.device
        alpha, ws_ptr, ws_len = float(self.alpha), None, 0
        if route == SPANNING:
            need = _hip.lib.ma_spanning_step_workspace(table.records, n, ctypes.byref(h))
            ws = self._workspace
            if ws is None or ws.numel() < need or ws.device != device:
                ws = self._workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
            ws_ptr, ws_len = ws.data_ptr(), ws.numel()
        if sums is not None:
            for e in entries:  # a logging step's kernels do not file the cuts of the row they write
                e.forget_row_cuts(e.st['index'])
            need = _hip.lib.ma_logged_step_partials(table.records, n, ctypes.byref(h))
            part = self._partials
            if part is None or part.numel() < need or part.device != device:
                part = self._partials = torch.empty(max(need, 8), dtype=torch.float32,
                                                    device=device)
            rc = _hip.lib.ma_logged_step(_LOGGED_ROUTE[route], table.records, n, ctypes.byref(h),
                                         alpha, ws_ptr, ws_len, part.data_ptr(), part.numel(),
                                         sums.data_ptr(), stream)
            _hip.check(rc, "ma_logged_step")
        elif route == FUSED:
            rc = _hip.lib.ma_fused_step(table.records, n, ctypes.byref(h), stream)
            _hip.check(rc, "ma_fused_step")
        elif route == FUSED_DENSIFIED:
            rc = _hip.lib.ma_fused_step_densified(table.records, n, ctypes.byref(h), alpha, stream)
            _hip.check(rc, "ma_fused_step_densified")
        elif route == FUSED_QUANT_ERR:
            rc = _hip.lib.ma_fused_step_quant_err(table.records, n, ctypes.byref(h), stream)
            _hip.check(rc, "ma_fused_step_quant_err")
        else:
            rc = _hip.lib.ma_spanning_step(table.records, n, ctypes.byref(h), alpha, ws_ptr,
                                           ws_len, stream)
            _hip.check(rc, "ma_spanning_step")
        for e in entries:  # micro_adam.py:211
            e.st['index'] = (e.st['index'] + 1) % self.m

    # ------------------------------------------------------------------ op-by-op route (micro_adam.py:146-328)
    @torch.no_grad()
    def update_step(self, p, lr, wd, logging_step=False):
        """One tensor through the reference's own sequence of device operations.  Returns the
        logging sums of this tensor (all zero unless logging_step)."""
        out = dict(norm_qe=0, norm_g=0, norm_u=0, norm_e=0, sparsity_u=0, sparsity_qe=0)
        entry = self._entry(p, lr, wd)
        st = entry.st
        entry.forget_row_cuts(st['index'])
        acc = p.grad.view(-1)  # the gradient buffer is accumulator, update and scratch in turn
        d, q = st['d'], self.quant_block_size
        error, lo, hi = st['error'], st['min_vals'], st['max_vals']
        stream, tag = _hip.stream_ptr(), _hip.dtype_tag(acc)
        acc_ptr = _hip.dev_ptr(acc, None, "grad")

        def add_dequantised(scale):  # acc += scale * Qinv(error)
            _ext_quant.asymm_block_quant_inv(d, q, error, lo, hi, acc, scale)

        def requantise():  # statistics of acc per quantisation block, then error = Q(acc)
            _hip.check(_hip.lib.ma_block_minmax(d, q, acc_ptr, _hip.dev_ptr(lo, torch.bfloat16, "min_vals"),
                                                _hip.dev_ptr(hi, torch.bfloat16, "max_vals"), tag,
                                                stream), "ma_block_minmax")
            _ext_quant.asymm_block_quant(d, q, error, lo, hi, acc)

        if logging_step:
            out['norm_g'] = acc.norm(p=2) ** 2

        # accumulator = gradient + error feedback; its block-wise top-k moves into window row
        # `index` (selection, value gather and zeroing are one launch); the rest is requantised
        add_dequantised(1.0)
        row = st['index']
        _hip.check(_hip.lib.ma_block_topk(d, st['d_block_size'], st['k_block_size_many'],
                                          st['k_block_size_few'], acc_ptr,
                                          _hip.dev_ptr(st['I'][row], torch.int16, "I row"),
                                          _hip.dev_ptr(st['V'][row], torch.bfloat16, "V row"),
                                          1, tag, stream), "ma_block_topk")
        st['index'] = (row + 1) % self.m
        requantise()

        # decoupled weight decay goes into the update kernel unless something reads p first
        plain = p.dtype == acc.dtype and p.is_contiguous()
        decay_in_kernel = plain and not self.densify_update_using_quant_error
        if wd > 0 and not decay_in_kernel:
            p.mul_(1 - lr * wd)

        if self.densify_update_using_quant_error:
            # alpha == -2 (micro_adam.py:238-273): what quantisation lost of the accumulator goes
            # straight into the parameters: p -= a, p += Qinv(Q(a)); quant_err keeps a - Qinv(Q(a))
            lost = st['quant_err']
            lost.copy_(p.grad)
            p.sub_(p.grad)
            acc.zero_()
            add_dequantised(1)
            p.add_(p.grad)
            lost.sub_(p.grad)
            if logging_step:
                out['norm_qe'] = lost.norm(p=2) ** 2
                out['sparsity_qe'] = (lost == 0).sum()

        # Adam direction rebuilt from the window, plus alpha * error feedback if asked for
        acc.zero_()
        _ext_quant.compute_microadam_update(st['blocks'], self.threads, self.shared_memory_carveout,
                                            self.steps, self.beta1, self.beta2, self.eps,
                                            st['d_block_size'], st['k_block_size_many'], d, self.m,
                                            st['k'], st['I'], st['V'], acc)
        if self.densify_update_using_ef:
            add_dequantised(self.alpha)

        if plain:
            decay = wd > 0 and decay_in_kernel
            _hip.check(_hip.lib.ma_param_update(d, _hip.dev_ptr(p, None, "p"), acc_ptr, -lr,
                                                1 if decay else 0, 1 - lr * wd, tag, stream),
                       "ma_param_update")
        else:
            p.add_(p.grad, alpha=-lr)

        if logging_step:
            out['norm_u'] = acc.norm(p=2) ** 2
            out['sparsity_u'] = (acc == 0).sum()

        if self.densify_update_using_ef:
            # the share of the error feedback that went into the update leaves it
            acc.zero_()
            add_dequantised(1 - self.alpha)
            requantise()

        if logging_step:
            acc.zero_()
            add_dequantised(1.0)
            out['norm_e'] = acc.norm(p=2) ** 2
        return out

    # ------------------------------------------------------------------ checkpointing
    def state_dict(self):
        """As torch's, plus the global step counter, which the reference keeps as a plain
        attribute (micro_adam.py:35) and therefore loses on resume: the ages of the window
        rows and the bias corrections depend on it."""
        sd = super().state_dict()
        sd['steps'] = self.steps
        return sd

    def load_state_dict(self, state_dict):
        """torch's load_state_dict casts all per-parameter tensors to the parameter's dtype,
        which would destroy int16 indices under bf16 parameters; the typed tensors are taken
        from the source dictionary again afterwards."""
        super().load_state_dict(state_dict)
        if 'steps' in state_dict:
            self.steps = int(state_dict['steps'])
        saved_ids = [pid for g in state_dict['param_groups'] for pid in g['params']]
        params = [p for g in self.param_groups for p in g['params']]
        for pid, p in zip(saved_ids, params):
            saved = state_dict['state'].get(pid)
            if saved is None:
                continue
            st = self.state[p]
            for key, dtype in _TYPED_STATE:
                if key in saved and torch.is_tensor(saved[key]) and saved[key].dtype == dtype:
                    st[key] = saved[key].to(device=p.device, copy=True)
        self._entries.clear()
        self._tables.clear()
        self._walk = None

    # ------------------------------------------------------------------ logging (micro_adam.py:330-350)
    @staticmethod
    def _logging_active():
        return wandb is not None and getattr(wandb, 'run', None) is not None

    def _log(self, norm_qe, norm_g, norm_u, norm_e, sparsity_u, sparsity_qe, elapsed_step):
        if self.steps % self.log_interval != 0:
            return
        sums = [norm_qe, norm_g, norm_u, norm_e, sparsity_u, sparsity_qe, elapsed_step]
        if _distributed():
            buf = torch.tensor([float(x) for x in sums], dtype=torch.float).cuda()
            dist.all_reduce(buf, op=dist.ReduceOp.SUM)
            sums = buf.tolist()
            if dist.get_rank() != 0:
                return
        norm_qe, norm_g, norm_u, norm_e, sparsity_u, sparsity_qe, elapsed_step = sums
        percent = 100. / self.model_size
        wandb.log({'step/optimizer_steps': self.steps,
                   'step/gpu_mem_usage': get_gpu_mem_usage(),
                   'step/norm_quant_err': math.sqrt(norm_qe),
                   'step/sparsity_quant_err': sparsity_qe * percent,
                   'step/norm_g': math.sqrt(norm_g),
                   'step/norm_u': math.sqrt(norm_u),
                   'step/norm_error': math.sqrt(norm_e),
                   'step/sparsity_u': sparsity_u * percent,
                   'step/elapsed_step': elapsed_step}, commit=False)
