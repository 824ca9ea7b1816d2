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


_F32 = torch.float32


def _prepare(online: Iterable[Optional[torch.Tensor]], target: Iterable[torch.Tensor], skip_none: bool):
    """Pairs the lists up as ``zip`` does, validates them and makes them dense.

    Written as a few flat comprehensions: at 150+ tensors per call the Python
    work here costs more than the kernel, so every per-tensor call counts."""
    pairs = list(zip(online, target))
    if any(s is None for s, _ in pairs):
        if not skip_none:
            raise TypeError("online parameter is None (use calculate_updated_momentum_encoder to skip those)")
        pairs = [p for p in pairs if p[0] is not None]  # benchmarks/moco-v3/main.py:139-140
    if not pairs:
        return [], []
    students = [s for s, _ in pairs]
    teachers = [t for _, t in pairs]
    dev = teachers[0].device
    if dev.type != "cuda":
        raise TypeError("EMA kernel needs device tensors (the pipeline asserts the same, tspipe/gpu_task.py:407)")
    if not all(t.dtype is _F32 and s.dtype is _F32 for s, t in pairs):
        bad = next((s.dtype, t.dtype) for s, t in pairs if not (t.dtype is _F32 and s.dtype is _F32))
        raise TypeError(f"EMA kernel is fp32 (got student {bad[0]}, teacher {bad[1]})")
    if not all(t.device == dev and s.device == dev for s, t in pairs):
        if any(not t.is_cuda or not s.is_cuda for s, t in pairs):
            raise TypeError("EMA kernel needs device tensors (the pipeline asserts the same, tspipe/gpu_task.py:407)")
        raise ValueError("teacher and student parameters live on different devices")
    if [t.shape for t in teachers] != [s.shape for s in students]:
        bad = next((tuple(t.shape), tuple(s.shape)) for s, t in pairs if t.shape != s.shape)
        raise ValueError(f"teacher/student shapes differ: {bad[0]} vs {bad[1]}")
    if not all(t.is_contiguous() and s.is_contiguous() for s, t in pairs):
        students = [s if s.is_contiguous() else s.detach().contiguous() for s in students]
        teachers = [t if t.is_contiguous() else t.detach().contiguous() for t in teachers]
    return students, teachers


def _launch(m: float, students: Sequence[torch.Tensor], teachers: Sequence[torch.Tensor],
            outs: Sequence[torch.Tensor], numels: np.ndarray) -> None:
    device = teachers[0].device
    with torch.cuda.device(device):
        table = _tables.stage_ema(_tables.ptr_array(teachers), _tables.ptr_array(students),
                                  _tables.ptr_array(outs), numels, device)
        timed = kernel_events is not None
        if timed:
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record(torch.cuda.current_stream(device))
        # the reference multiplies by the Python doubles m and (1. - m); torch
        # rounds each to fp32 before the fp32 multiply, and so does ctypes here
        status = _lib.lib().ts_ema_multi(table.dev_ptr, table.n_chunks, table.chunk, float(m), 1.0 - float(m),
                                        _lib.current_stream_ptr(device))
        _lib.check(status, "ts_ema_multi")
        if timed:
            end.record(torch.cuda.current_stream(device))
            kernel_events.append((start, end))
        table.done()


def _new_outputs(teachers: Sequence[torch.Tensor], numels: np.ndarray) -> List[torch.Tensor]:
    """One flat allocation carved into views shaped like the teachers, each
    starting on a 16-byte boundary."""
    device = teachers[0].device
    if not (numels & 3).any():
        # every size is a multiple of 4 elements: pieces are back to back and
        # torch's C++ unflatten makes all the views in one call
        flat = torch.empty(int(numels.sum()), dtype=_F32, device=device)
        return list(torch._C._nn.unflatten_dense_tensors(flat, teachers))
    padded = ((numels + 3) & ~3).tolist()
    flat = torch.empty(sum(padded), dtype=_F32, device=device)
    pieces = flat.split(padded)
    return [p[:t.numel()].view(t.shape) for p, t in zip(pieces, teachers)]


@torch.no_grad()
def momentum_update(m: float, online_new_param: Iterable[Optional[torch.Tensor]],
                    target_param: Iterable[torch.Tensor], skip_none: bool = False) -> List[torch.Tensor]:
    """Returns new tensors ``t*m + s*(1-m)``; the inputs are left untouched."""
    students, teachers = _prepare(online_new_param, target_param, skip_none)
    if not teachers:
        return []
    numels = np.fromiter((t.numel() for t in teachers), dtype=np.int64, count=len(teachers))
    outs = _new_outputs(teachers, numels)
    _launch(m, students, teachers, outs, numels)
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
    numels = np.fromiter((t.numel() for t in teachers), dtype=np.int64, count=len(teachers))
    _launch(m, students, teachers, teachers, numels)
    for live, work in zip(target_params, teachers):
        if work.data_ptr() != live.data_ptr():  # a non-contiguous parameter was densified
            live.detach().copy_(work)
