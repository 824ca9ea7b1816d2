"""Momentum-teacher EMA over a whole parameter list in one HIP launch.

Drop-in for TSPipe's ``target_update_fn`` plug-in, which the pipeline calls as
``fn(momentum, online_new_param, target_prev_param)`` and whose result it stores
as a new parameter version (tspipe/gpu_task.py:403-410).  The two reference
implementations of that plug-in are
``TSPipeBYOLTrainer.calculate_target_network_parameters``
(benchmarks/byol/trainer.py:198-212) and ``calculate_updated_momentum_encoder``
(benchmarks/moco-v3/main.py:133-144): per tensor,
``t.clone() * m + s * (1. - m)``, returned as a new list.
"""
from typing import Iterable, List, Optional, Sequence

import numpy as np
import torch

from . import _lib, _tables

# When set to a list, every EMA launch appends a (start, end) pair of HIP
# events recorded on the launch stream around the kernel alone (profiling aid).
kernel_events = None


def _prepare(online: Iterable[Optional[torch.Tensor]], target: Iterable[torch.Tensor], skip_none: bool):
    students, teachers = [], []
    for s, t in zip(online, target):
        if s is None:
            if skip_none:
                continue  # benchmarks/moco-v3/main.py:139-140
            raise TypeError("online parameter is None (use calculate_updated_momentum_encoder to skip those)")
        s, t = s.detach(), t.detach()
        if t.shape != s.shape:
            raise ValueError(f"teacher/student shapes differ: {tuple(t.shape)} vs {tuple(s.shape)}")
        if t.dtype != torch.float32 or s.dtype != torch.float32:
            raise TypeError(f"EMA kernel is fp32 (got teacher {t.dtype}, student {s.dtype})")
        if not t.is_cuda or not s.is_cuda:
            raise TypeError("EMA kernel needs device tensors (the pipeline asserts the same, tspipe/gpu_task.py:407)")
        if t.device != s.device:
            raise ValueError("teacher and student live on different devices")
        students.append(s if s.is_contiguous() else s.contiguous())
        teachers.append(t if t.is_contiguous() else t.contiguous())
    return students, teachers


def _launch(m: float, students: Sequence[torch.Tensor], teachers: Sequence[torch.Tensor],
            outs: Sequence[torch.Tensor]) -> None:
    device = teachers[0].device
    numels = np.fromiter((t.numel() for t in teachers), dtype=np.int64, count=len(teachers))
    with torch.cuda.device(device):
        table = _tables.stage_ema(_tables.ptr_array(teachers), _tables.ptr_array(students),
                                  _tables.ptr_array(outs), numels, device)
        # the reference multiplies by the Python doubles m and (1. - m); torch
        # rounds each to fp32 before the fp32 multiply
        timed = kernel_events is not None
        if timed:
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record(torch.cuda.current_stream(device))
        status = _lib.lib().ts_ema_multi(table.dev_ptr, table.n_chunks, float(m), 1.0 - float(m),
                                        _lib.current_stream_ptr(device))
        _lib.check(status, "ts_ema_multi")
        if timed:
            end.record(torch.cuda.current_stream(device))
            kernel_events.append((start, end))
        table.done()


def _new_outputs(teachers: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    """One flat allocation, carved into 16-byte aligned views shaped like the teachers."""
    padded = [(t.numel() + 3) & ~3 for t in teachers]
    flat = torch.empty(sum(padded), dtype=torch.float32, device=teachers[0].device)
    pieces = flat.split(padded)
    return [p[:t.numel()].view(t.shape) if p.numel() != t.numel() else p.view(t.shape)
            for p, t in zip(pieces, teachers)]


@torch.no_grad()
def momentum_update(m: float, online_new_param: Iterable[Optional[torch.Tensor]],
                    target_param: Iterable[torch.Tensor], skip_none: bool = False) -> List[torch.Tensor]:
    """Returns new tensors ``t*m + s*(1-m)``; the inputs are left untouched."""
    students, teachers = _prepare(online_new_param, target_param, skip_none)
    if not teachers:
        return []
    outs = _new_outputs(teachers)
    _launch(m, students, teachers, outs)
    return outs


def calculate_target_network_parameters(m, online_new_param, target_param=None):
    """BYOL plug-in (benchmarks/byol/trainer.py:198-212)."""
    return momentum_update(m, online_new_param, target_param, skip_none=False)


def calculate_updated_momentum_encoder(m, online_param, momentum_encoder):
    """MoCo-v3 plug-in (benchmarks/moco-v3/main.py:133-144): ``None`` student entries are skipped."""
    return momentum_update(m, online_param, momentum_encoder, skip_none=True)


@torch.no_grad()
def update_target_network_parameters_(online_params: Iterable[torch.Tensor],
                                      target_params: Iterable[torch.Tensor], m: float) -> None:
    """In-place form used by the non-pipelined training loops:
    ``param_k.data = param_k.data * m + param_q.data * (1. - m)``
    (benchmarks/byol/trainer.py:43-49, benchmarks/moco-v3/moco/builder.py:57-61)."""
    target_params = list(target_params)
    students, teachers = _prepare(online_params, target_params, skip_none=False)
    if not teachers:
        return
    _launch(m, students, teachers, teachers)
    for live, work in zip(target_params, teachers):
        if work.data_ptr() != live.data_ptr():  # a non-contiguous parameter was densified
            live.detach().copy_(work)
