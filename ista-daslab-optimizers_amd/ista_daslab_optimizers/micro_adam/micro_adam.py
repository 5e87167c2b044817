"""MicroAdam on MI355X: the optimizer of ista_daslab_optimizers/micro_adam/micro_adam.py with
the same constructor, attributes and per-parameter state, driving gfx950 HIP kernels through
libmicroadam_hip.so.

Two routes compute the same step (reference micro_adam.py:146-328):
  * fused: one kernel pass per top-k block does Qinv + add, block top-k, window write,
    requantisation, window -> Adam direction and the parameter update.  Taken for tensors
    the kernel's layout conditions admit (see ma_fused_step in include/microadam_hip.h)
    when alpha == 0.
  * op by op: the reference's own sequence of extension calls, each a HIP kernel, with the
    stock torch ops of the sequence (abs/topk, min/max, add_) replaced by kernels as well.
    Taken for everything else (alpha > 0, alpha == -2, odd quantisation block sizes,
    logging steps).
There is no CPU or pure-PyTorch route; a missing library or a CPU tensor raises.
"""
import ctypes
import math
import time

import torch
from torch.distributed import is_initialized, get_rank, all_reduce, ReduceOp

import ista_daslab_cuda_micro_adam
import ista_daslab_cuda_tools

from .. import _hip
from ..tools import get_first_device, get_gpu_mem_usage, block_split, CopyDirection

try:  # logging is optional here; the reference imports wandb unconditionally (micro_adam.py:5)
    import wandb
except Exception:  # pragma: no cover
    wandb = None


class MicroAdam(torch.optim.Optimizer):
    def __init__(self, params, m, lr, quant_block_size, k_init=0.01, alpha=0, betas=(0.9, 0.999),
                 weight_decay=0, eps=1e-8):
        defaults = dict(lr=lr, weight_decay=weight_decay, eps=eps, alpha=alpha)
        super(MicroAdam, self).__init__(params, defaults)

        assert (0 <= alpha < 1) or alpha == -2, 'Alpha must be in the [0, 1) interval or -2'

        self.m = m
        self.lr = lr
        self.quant_block_size = int(quant_block_size)
        self.k_init = k_init
        self.alpha = alpha
        self.weight_decay = weight_decay
        self.beta1 = betas[0]
        self.beta2 = betas[1]
        self.eps = eps

        self.densify_update_using_ef = (self.alpha > 0)
        self.densify_update_using_quant_error = (self.alpha == -2)

        self.model_size = sum([p.numel() for group in self.param_groups for p in group['params']])

        self.steps = 0  # how many optimization steps were performed so far
        self.log_interval = 100
        self.device = get_first_device()
        self._is_state_initialized = False
        self.shared_memory_carveout = 100
        self.blocks = ista_daslab_cuda_tools.get_sm_count() * int(100 / self.shared_memory_carveout)
        self.threads = 512

        self.max_floats = ista_daslab_cuda_tools.get_max_floats_for_shared_memory_per_thread_block()
        self.d_block_size = self.max_floats // 2 // int(100 / self.shared_memory_carveout)

        if torch.distributed.is_available() and torch.distributed.is_initialized():
            self.fsdp_dict_size_count = [{} for _ in range(torch.distributed.get_world_size())]
        else:
            self.fsdp_dict_size_count = [{}]

        self.dict_size_count = {}  # key = layer size, value = how many layers of that size the model has
        for param in self.param_groups:
            for p in param['params']:
                size = p.numel()
                self.dict_size_count[size] = 1 + self.dict_size_count.get(size, 0)

        # not in the reference: route selection and the cached descriptor table of the fused step
        self.use_fused = True
        self._fused_cache = None
        self._route = {}
        self._workspace = None  # device scratch of the spanning route, grown on demand

    # ------------------------------------------------------------------ state (micro_adam.py:61-94)
    def _initialize_parameter_state(self, p, lr, wd):
        layer_size = p.numel()
        st = self.state[p]

        rank = torch.distributed.get_rank() if (torch.distributed.is_available() and torch.distributed.is_initialized()) else 0

        if self.densify_update_using_quant_error:
            st['quant_err'] = torch.zeros_like(p)

        count = self.fsdp_dict_size_count[rank].get(layer_size, 1)
        st['blocks'] = max(1, int(math.floor(self.blocks * layer_size * count / self.model_size)))

        st['lr'] = lr
        st['weight_decay'] = wd
        st['d'] = layer_size

        ##### variables for Top-K: d_index_topk is the index where the last, smaller topk block starts
        st['d_block_size'] = layer_size if layer_size < self.d_block_size else self.d_block_size
        st['topk_full_blocks_count'], st['d_index_topk'] = block_split(st['d'], st['d_block_size'])
        st['k_block_size_many'] = int(math.ceil(st['d_block_size'] * self.k_init))
        st['k_block_size_few'] = int(math.ceil((st['d'] - st['d_index_topk']) * self.k_init))  # 0 for d % self.d_block_size = 0
        st['k_index'] = st['topk_full_blocks_count'] * st['k_block_size_many']
        st['k'] = st['k_block_size_many'] * st['topk_full_blocks_count'] + st['k_block_size_few']

        ##### variables for the ring buffer
        st['index'] = 0  # the position to place a new gradient at
        st['I'] = torch.zeros(self.m, st['k'], dtype=torch.int16, device=p.device)  # 2mk bytes
        st['V'] = torch.zeros(self.m, st['k'], dtype=torch.bfloat16, device=p.device)  # 2mk bytes

        ### variables for error feedback: d_index_quant is the index where the last, smaller quantization block starts
        st['quant_full_blocks_count'], st['d_index_quant'] = block_split(st['d'], self.quant_block_size)
        st['error'] = torch.zeros(int(math.ceil(st['d'] / 2)), dtype=torch.uint8, device=p.device)  # ceil(d/2) bytes
        st['min_vals'] = torch.zeros(st['quant_full_blocks_count'] + 1, dtype=torch.bfloat16, device=p.device)
        st['max_vals'] = torch.zeros(st['quant_full_blocks_count'] + 1, dtype=torch.bfloat16, device=p.device)

    # ------------------------------------------------------------------ step (micro_adam.py:96-144)
    @torch.no_grad()
    def step(self, closure=None):
        self.steps += 1

        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        if self.steps == 1:
            rank = torch.distributed.get_rank() if (torch.distributed.is_available() and torch.distributed.is_initialized()) else 0
            for param in self.param_groups:
                for p in param['params']:
                    if p is not None:
                        size = p.numel()
                        if size > 0:
                            self.fsdp_dict_size_count[rank][size] = 1 + self.fsdp_dict_size_count[rank].get(size, 0)

        time_start = time.time()

        norm_qe, norm_g, norm_u, norm_e, sparsity_u, sparsity_qe = 0, 0, 0, 0, 0, 0
        logging_step = self._logging_active() and self.steps % self.log_interval == 0

        fused, spanning, dense = [], [], []  # (p, st, lr, wd)
        log_after = []  # tensors a fused kernel steps on a logging step: metrics taken afterwards
        for group in self.param_groups:
            lr = group['lr']
            wd = group.get('weight_decay', self.weight_decay)

            for p in group['params']:
                if p.grad is None:
                    continue

                if p is None:
                    continue

                st = self.state[p]
                if len(st) == 0:
                    self._check_param(p)
                    self._initialize_parameter_state(p, lr, wd)
                self._repair_state(st)

                route = self._fusable(p, st) if self.use_fused else 0
                if logging_step and not (route in (1, 2) and self.alpha == 0):
                    # with alpha != 0 the update holds a term that no state keeps: op by op
                    route = 0
                if route:
                    if logging_step:
                        norm_g += p.grad.view(-1).norm(p=2) ** 2  # the spanning route overwrites g
                        log_after.append((p, st))
                    (fused, spanning, dense)[route - 1].append((p, st, lr, wd))
                    continue

                nqe, ng, nu, ne, sp_u, sp_qe = self.update_step(p, lr, wd, logging_step)
                norm_qe += nqe
                norm_g += ng
                norm_u += nu
                norm_e += ne
                sparsity_u += sp_u
                sparsity_qe += sp_qe

        if fused:
            self._fused_step(fused)
        if spanning:
            self._fused_step(spanning, spanning=True)
        if dense:
            self._fused_step(dense, dense=True)
        for p, st in log_after:
            nu, ne, sp_u = self._metrics_after_fused_step(p, st)
            norm_u += nu
            norm_e += ne
            sparsity_u += sp_u

        time_end = time.time()
        elapsed_step = time_end - time_start
        if logging_step:
            self._log(norm_qe, norm_g, norm_u, norm_e, sparsity_u, sparsity_qe, elapsed_step)

        return loss

    # ------------------------------------------------------------------ fused route
    @staticmethod
    def _check_param(p):
        if not p.is_cuda:
            raise RuntimeError(f"MicroAdam runs on the GPU only; got a parameter on {p.device}")
        if p.dtype not in (torch.float32, torch.bfloat16):
            raise TypeError(f"MicroAdam takes float32 or bfloat16 parameters, got {p.dtype}")

    _STATE_DTYPES = (('I', torch.int16), ('V', torch.bfloat16), ('error', torch.uint8),
                     ('min_vals', torch.bfloat16), ('max_vals', torch.bfloat16))

    @classmethod
    def _repair_state(cls, st):
        # Frameworks that reload or re-type optimizer state cast every state tensor to the
        # parameter's dtype (the reference repairs st['I'] for this reason,
        # micro_adam.py:175-178); the kernels need the declared types back.
        for key, dtype in cls._STATE_DTYPES:
            if st[key].dtype != dtype:
                st[key] = st[key].to(dtype)

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
            for key, dtype in self._STATE_DTYPES:
                if key in saved and torch.is_tensor(saved[key]) and saved[key].dtype == dtype:
                    st[key] = saved[key].to(device=p.device, copy=True)
        self._fused_cache = None

    def _fusable(self, p, st):
        """0: op-by-op route; 1: ma_fused_step (alpha == 0, quantisation blocks inside the top-k
        blocks); 2: ma_spanning_step (0 <= alpha < 1, quantisation blocks at least as long as the
        top-k blocks); 3: ma_fused_step_densified (as 1 with 0 < alpha < 1).  The conditions are
        those of include/microadam_hip.h."""
        if not 0 <= self.alpha < 1:
            return 0
        g = p.grad
        if g.dtype != p.dtype or not p.is_contiguous() or not g.is_contiguous():
            return 0
        if (p.data_ptr() | g.data_ptr()) & 15:
            return 0
        route = self._route.get(id(p))
        if route is None:
            q, d, dbs = self.quant_block_size, st['d'], st['d_block_size']
            common = (self.m <= _hip.MA_MAX_WINDOW and dbs <= 32768
                      and (d <= self.d_block_size or dbs % 8 == 0))
            route = 0
            if (common and 8 <= q <= 512 and (q & (q - 1)) == 0 and d >= q
                    and (d <= self.d_block_size or dbs % q == 0)):
                route = 1 if self.alpha == 0 else 3
            elif (common and q % 8 == 0 and dbs <= q < (1 << 30)
                  and (q + dbs - 1) // dbs + 1 <= 64):
                route = 2
            self._route[id(p)] = route
        return route

    def _fused_step(self, items, spanning=False, dense=False):
        n = len(items)
        kind = 1 if spanning else 2 if dense else 0
        key = (kind,) + tuple(id(p) for p, _, _, _ in items)
        cache = self._fused_cache.get(kind) if self._fused_cache else None
        if cache is None or cache[0] != key:
            arr = (_hip.MaTensor * n)()
            for t, (p, st, _, _) in zip(arr, items):
                t.d = st['d']
                t.k = st['k']
            cache = (key, arr)
            if self._fused_cache is None:
                self._fused_cache = {}
            self._fused_cache[kind] = cache
        arr = cache[1]
        for t, (p, st, lr, wd) in zip(arr, items):
            t.p = p.data_ptr()
            t.g = p.grad.data_ptr()
            t.error = st['error'].data_ptr()
            t.min_vals = st['min_vals'].data_ptr()
            t.max_vals = st['max_vals'].data_ptr()
            t.I = st['I'].data_ptr()
            t.V = st['V'].data_ptr()
            t.lr = lr
            t.weight_decay = wd
            t.index = st['index']
        by_dtype = {}
        for i, (p, _, _, _) in enumerate(items):
            by_dtype.setdefault(p.dtype, []).append(i)
        for dtype, idxs in by_dtype.items():
            if len(idxs) == n:
                sub, cnt = arr, n
            else:
                sub = (_hip.MaTensor * len(idxs))(*[arr[i] for i in idxs])
                cnt = len(idxs)
            h = _hip.MaHyper(self.steps, self.m, _hip.MA_BF16 if dtype == torch.bfloat16 else _hip.MA_F32,
                             self.quant_block_size, self.d_block_size, self.k_init, self.beta1,
                             self.beta2, self.eps)
            if dense:
                rc = _hip.lib.ma_fused_step_densified(sub, cnt, ctypes.byref(h), float(self.alpha),
                                                      _hip.stream_ptr())
                _hip.check(rc, "ma_fused_step_densified")
                continue
            if not spanning:
                rc = _hip.lib.ma_fused_step(sub, cnt, ctypes.byref(h), _hip.stream_ptr())
                _hip.check(rc, "ma_fused_step")
                continue
            need = _hip.lib.ma_spanning_step_workspace(sub, cnt, ctypes.byref(h))
            ws = self._workspace
            if ws is None or ws.numel() < need or ws.device != items[idxs[0]][0].device:
                ws = self._workspace = torch.empty(max(need, 16), dtype=torch.uint8,
                                                   device=items[idxs[0]][0].device)
            rc = _hip.lib.ma_spanning_step(sub, cnt, ctypes.byref(h), float(self.alpha),
                                            ws.data_ptr(), ws.numel(), _hip.stream_ptr())
            _hip.check(rc, "ma_spanning_step")
        for _, st, _, _ in items:
            st['index'] = (st['index'] + 1) % self.m

    # ------------------------------------------------------------------ op-by-op route (micro_adam.py:146-328)
    @torch.no_grad()
    def update_step(self, p, lr, wd, logging_step=False):
        norm_qe, norm_g, norm_u, norm_e, sp_u, sp_qe = 0, 0, 0, 0, 0, 0

        grad = p.grad.view(-1)

        if logging_step:
            norm_g = grad.norm(p=2) ** 2

        st = self.state[p]
        if len(st) == 0:
            self._check_param(p)
            self._initialize_parameter_state(p, lr, wd)

        blocks = st['blocks']
        d = st['d']
        d_block_size = st['d_block_size']
        k_block_size_many = st['k_block_size_many']
        k_block_size_few = st['k_block_size_few']
        k = st['k']

        self._repair_state(st)

        index = st['index']
        I = st['I']
        V = st['V']

        error = st['error']
        min_vals = st['min_vals']
        max_vals = st['max_vals']
        stream = _hip.stream_ptr()
        tag = _hip.dtype_tag(grad)
        gptr = _hip.dev_ptr(grad, None, "grad")

        ##### STEP 4
        ista_daslab_cuda_micro_adam.asymm_block_quant_inv(d, self.quant_block_size, error, min_vals, max_vals, grad, 1.0)

        ##### STEP 5 + 9 + 6: block top-k, V = a[I], a[I] = 0 in one launch
        _hip.check(_hip.lib.ma_block_topk(d, d_block_size, k_block_size_many, k_block_size_few, gptr,
                                          _hip.dev_ptr(I[index, :], torch.int16, "I row"),
                                          _hip.dev_ptr(V[index, :], torch.bfloat16, "V row"),
                                          1, tag, stream), "ma_block_topk")

        st['index'] = (index + 1) % self.m

        ##### STEP 7
        def _update_quantization_statistics():
            _hip.check(_hip.lib.ma_block_minmax(d, self.quant_block_size, gptr,
                                                _hip.dev_ptr(min_vals, torch.bfloat16, "min_vals"),
                                                _hip.dev_ptr(max_vals, torch.bfloat16, "max_vals"),
                                                tag, stream), "ma_block_minmax")

        _update_quantization_statistics()

        ##### STEP 8
        ista_daslab_cuda_micro_adam.asymm_block_quant(d, self.quant_block_size, error, min_vals, max_vals, grad)  # error = Q(a, min, max)

        # weight decay step: folded into the update kernel below unless something reads p first
        same_layout = p.dtype == grad.dtype and p.is_contiguous()
        fold_decay = same_layout and not self.densify_update_using_quant_error
        if wd > 0 and not fold_decay:
            p.mul_(1 - lr * wd)

        ##### NEW: densify using quant error (micro_adam.py:238-273)
        if self.densify_update_using_quant_error:
            quant_err = st['quant_err']
            quant_err.zero_()
            quant_err.add_(p.grad)

            ##### STEP A
            p.add_(p.grad, alpha=-1)

            ##### STEP B
            p.grad.zero_()  # zerorize to prepare the accumulator for Qinv
            ista_daslab_cuda_micro_adam.asymm_block_quant_inv(d, self.quant_block_size, error, min_vals, max_vals, grad, 1)
            p.add_(p.grad)

            quant_err.sub_(p.grad)

            if logging_step:
                norm_qe = quant_err.norm(p=2) ** 2
                sp_qe = (quant_err == 0).sum()

        ##### STEPS 10-11
        grad.zero_()
        ista_daslab_cuda_micro_adam.compute_microadam_update(blocks,  # blocks
                                                             self.threads,  # threads
                                                             self.shared_memory_carveout,  # carveout
                                                             self.steps,  # optimization step
                                                             self.beta1,  # beta1
                                                             self.beta2,  # beta2
                                                             self.eps,  # eps
                                                             d_block_size,  # d_block_size
                                                             k_block_size_many,  # k_block_size
                                                             d,  # d
                                                             self.m,  # m
                                                             k,  # k
                                                             I,  # indices
                                                             V,  # values
                                                             grad)  # update will be stored here

        ##### if PRETRAINING #1
        if self.densify_update_using_ef:  # we add alpha * EF to update that is stored in grad buffer
            ista_daslab_cuda_micro_adam.asymm_block_quant_inv(d, self.quant_block_size, error, min_vals, max_vals, grad, self.alpha)

        # update model using MicroAdam update stored in p.grad
        if same_layout:
            apply_decay = wd > 0 and fold_decay
            _hip.check(_hip.lib.ma_param_update(d, _hip.dev_ptr(p, None, "p"), gptr, -lr,
                                                1 if apply_decay else 0, 1 - lr * wd, tag, stream),
                       "ma_param_update")
        else:
            p.add_(p.grad, alpha=-lr)

        if logging_step:
            norm_u = grad.norm(p=2) ** 2
            sp_u = (grad == 0).sum()  # check sparsity before zerorizing

        ##### if PRETRAINING #2
        if self.densify_update_using_ef:
            grad.zero_()
            ista_daslab_cuda_micro_adam.asymm_block_quant_inv(d, self.quant_block_size, error, min_vals, max_vals, grad, 1 - self.alpha)

            _update_quantization_statistics()  # step 7 again
            ista_daslab_cuda_micro_adam.asymm_block_quant(d, self.quant_block_size, error, min_vals, max_vals, grad)  # step 8 again

        # compute error norm
        if logging_step:
            grad.zero_()
            ista_daslab_cuda_micro_adam.asymm_block_quant_inv(d, self.quant_block_size, error, min_vals, max_vals, grad, 1.0)

            norm_e = grad.norm(p=2) ** 2

        return norm_qe, norm_g, norm_u, norm_e, sp_u, sp_qe

    def _metrics_after_fused_step(self, p, st):
        """norm_u, norm_e and the update's zero count (micro_adam.py:306-308, :320-324) for a
        tensor that a fused kernel has just stepped with alpha == 0: the update is rebuilt from
        the window (which already holds this step's row, as at micro_adam.py:277-291) and the
        error norm from the stored error feedback, both in p.grad, which the step leaves as
        scratch like the reference does (:276, :321)."""
        grad = p.grad.view(-1)
        d = st['d']
        grad.zero_()
        ista_daslab_cuda_micro_adam.compute_microadam_update(
            st['blocks'], self.threads, self.shared_memory_carveout, self.steps, self.beta1,
            self.beta2, self.eps, st['d_block_size'], st['k_block_size_many'], d, self.m, st['k'],
            st['I'], st['V'], grad)
        norm_u = grad.norm(p=2) ** 2
        sp_u = (grad == 0).sum()
        grad.zero_()
        ista_daslab_cuda_micro_adam.asymm_block_quant_inv(d, self.quant_block_size, st['error'],
                                                          st['min_vals'], st['max_vals'], grad, 1.0)
        norm_e = grad.norm(p=2) ** 2
        return norm_u, norm_e, sp_u

    # ------------------------------------------------------------------ logging (micro_adam.py:330-350)
    @staticmethod
    def _logging_active():
        return wandb is not None and getattr(wandb, 'run', None) is not None

    def _log(self, norm_qe, norm_g, norm_u, norm_e, sparsity_u, sparsity_qe, elapsed_step):
        if self.steps % self.log_interval == 0:
            if is_initialized():
                sync_data = torch.tensor([norm_qe, norm_g, norm_u, norm_e, sparsity_u, sparsity_qe, elapsed_step], dtype=torch.float,
                                         requires_grad=False).cuda()
                all_reduce(sync_data, op=ReduceOp.SUM)
                norm_qe, norm_g, norm_u, norm_e, sparsity_u, sparsity_qe, elapsed_step = sync_data

            if not is_initialized() or get_rank() == 0:
                wandb_data = {
                    'step/optimizer_steps': self.steps,
                    'step/gpu_mem_usage': get_gpu_mem_usage(),
                    'step/norm_quant_err': math.sqrt(norm_qe),
                    'step/sparsity_quant_err': sparsity_qe / self.model_size * 100.,
                    'step/norm_g': math.sqrt(norm_g),
                    'step/norm_u': math.sqrt(norm_u),
                    'step/norm_error': math.sqrt(norm_e),
                    'step/sparsity_u': sparsity_u / self.model_size * 100.,
                    'step/elapsed_step': elapsed_step,
                }
                wandb.log(wandb_data, commit=False)
