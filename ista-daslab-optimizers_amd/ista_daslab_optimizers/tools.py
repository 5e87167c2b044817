"""Host helpers of the MicroAdam path, mirroring ista_daslab_optimizers/tools.py."""
import os
from enum import Enum

import torch


class CopyDirection(Enum):
    """tools.py:12-14"""
    k2d = 0
    d2k = 1


def get_first_device():
    """tools.py:29-34"""
    if not torch.cuda.is_available():
        return torch.device('cpu')
    if torch.distributed.is_available() and torch.distributed.is_initialized():
        return torch.device(f'cuda:{torch.distributed.get_rank()}')
    return torch.device('cuda:0')


def block_split(model_size, block_size):
    """tools.py:85-92: number of full blocks and the start of the last, shorter one."""
    if model_size < block_size:
        return 1, model_size
    blocks_count = int(model_size / block_size)
    start_index_last_block = model_size - model_size % block_size
    return blocks_count, start_index_last_block


def get_gpu_mem_usage():
    """tools.py:49-83 reports this process's GPU memory through gpustat; without gpustat
    the figure comes from torch's allocator, in MiB."""
    try:
        import gpustat
        gpus = gpustat.new_query().gpus
        gids = list(map(int, os.environ['CUDA_VISIBLE_DEVICES'].split(',')))
        return sum(int(proc['gpu_memory_usage']) for gid in gids for proc in gpus[gid]['processes']
                   if int(proc['pid']) == os.getpid())
    except Exception:
        if torch.cuda.is_available():
            return torch.cuda.memory_allocated() // (1 << 20)
        return 0
