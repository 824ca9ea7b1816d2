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
import operator
import sys
import threading
import weakref
from typing import Iterable, List, Optional, Sequence

import numpy as np
import torch

from . import _lib, _tables

# When set to a list, every EMA launch appends a (start, end) pair of HIP
# events stamped with the kernel's own begin and end (profiling aid).
kernel_events = None


_F32 = torch.float32
# the dtype codes of the C ABI (ts_dtype)
_DTYPE_CODES = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
_shape_of = operator.attrgetter("shape")
_dtype_of = operator.attrgetter("dtype")
_device_of = operator.attrgetter("device")
_use_count = getattr(torch._C, "_storage_Use_Count", None)


def _prepare(online: Iterable[Optional[torch.Tensor]], target: Iterable[torch.Tensor], skip_none: bool):
    """Pairs the lists up as ``zip`` does, validates them and makes them dense.
    Returns (students, teachers, shapes).

    At 150+ tensors per call the Python work here costs more than the kernel,
    so the checks run as C-level ``map`` calls over the lists rather than as a
    Python loop per tensor."""
    pairs = list(zip(online, target))
    if any(s is None for s, _ in pairs):
        if not skip_none:
            raise TypeError("online parameter is None (use calculate_updated_momentum_encoder to skip those)")
        pairs = [p for p in pairs if p[0] is not None]  # benchmarks/moco-v3/main.py:139-140
    if not pairs:
        return [], [], ()
    students = [p[0] for p in pairs]
    teachers = [p[1] for p in pairs]
    devices = set(map(_device_of, teachers)) | set(map(_device_of, students))
    if len(devices) != 1:
        if any(d.type != "cuda" for d in devices):
            raise TypeError("EMA kernel needs device tensors (the pipeline asserts the same, tspipe/gpu_task.py:407)")
        raise ValueError("teacher and student parameters live on different devices")
    if next(iter(devices)).type != "cuda":
        raise TypeError("EMA kernel needs device tensors (the pipeline asserts the same, tspipe/gpu_task.py:407)")
    dtypes = set(map(_dtype_of, teachers)) | set(map(_dtype_of, students))
    if len(dtypes) != 1 or next(iter(dtypes)) not in _DTYPE_CODES:
        raise TypeError(f"EMA kernel takes one of fp32 / bf16 / fp16 for all tensors (got {sorted(map(str, dtypes))})")
    shapes = tuple(map(_shape_of, teachers))
    if shapes != tuple(map(_shape_of, students)):
        bad = next((tuple(t.shape), tuple(s.shape)) for s, t in pairs if t.shape != s.shape)
        raise ValueError(f"teacher/student shapes differ: {bad[0]} vs {bad[1]}")
    if not (all(map(torch.Tensor.is_contiguous, teachers)) and all(map(torch.Tensor.is_contiguous, students))):
        students = [s if s.is_contiguous() else s.detach().contiguous() for s in students]
        teachers = [t if t.is_contiguous() else t.detach().contiguous() for t in teachers]
    return students, teachers, shapes


def _ptrs(tensors: Sequence[torch.Tensor]) -> np.ndarray:
    return np.array(list(map(torch.Tensor.data_ptr, tensors)), dtype=np.uint64)


def _launch(m: float, students: Sequence[torch.Tensor], teachers: Sequence[torch.Tensor],
            out_ptrs: np.ndarray, numels: np.ndarray) -> None:
    device = teachers[0].device
    code = _DTYPE_CODES[teachers[0].dtype]
    with _lib.on_device(device):
        table = _tables.stage_ema(_ptrs(teachers), _ptrs(students), out_ptrs, numels, device, dtype=code)
        timed = kernel_events is not None
        if timed:
            start, end = _lib.time_next_launch(device)
        # the reference multiplies by the Python doubles m and (1. - m); torch
        # rounds each to fp32 before the multiply (also for 2-byte tensors,
        # whose products are formed in fp32), and so does ctypes here
        if code == 0:
            status = _lib.lib().ts_ema_multi(table.dev_ptr, table.n_chunks, table.chunk, float(m), 1.0 - float(m),
                                            _lib.current_stream_ptr(device))
        else:
            status = _lib.lib().ts_ema_multi_dtype(table.dev_ptr, table.n_chunks, table.chunk, float(m),
                                                  1.0 - float(m), code, _lib.current_stream_ptr(device))
        _lib.check(status, "ts_ema_multi")
        if timed:
            kernel_events.append((start, end))
        table.done()


_tls = threading.local()


def _scratch(n: int):
    """Per-thread pointer / size arrays the C++ helper fills."""
    buf = getattr(_tls, "buf", None)
    if buf is None or buf[0].size < n:
        cap = max(256, 2 * n)
        buf = _tls.buf = (np.empty(cap, np.uint64), np.empty(cap, np.uint64), np.empty(cap, np.int64))
    return buf


def _fast_update(m: float, online, target) -> Optional[List[torch.Tensor]]:
    """The common case -- two lists of dense fp32 tensors on one GPU -- with the
    per-tensor work done by the C++ helper.  Returns None whenever anything is
    unusual (no helper, not lists, None entries, strided tensors, errors): the
    Python path then handles it or raises the proper exception."""
    host = _lib.host_helper()
    if host is None or type(online) is not list or type(target) is not list or _use_count is None:
        return None
    n = min(len(online), len(target))
    if n == 0:
        return None
    sp, tp, nn = _scratch(n)
    status, n, dev_index, shape_hash, total = host.pair_info(online, target, sp.ctypes.data, tp.ctypes.data,
                                                             nn.ctypes.data, sp.size)
    if status != 0:
        return None
    teachers = target if len(target) == n else target[:n]
    arena, views = _acquire_arena(teachers, (n, total, shape_hash))
    if arena.numels.size != n or not np.array_equal(arena.numels, nn[:n]):
        return None  # hash collision between different lists: take the exact path
    device = teachers[0].device
    with _lib.on_device(device):
        table = _tables.stage_ema(tp[:n], sp[:n], arena.ptrs, arena.numels, device)
        timed = kernel_events is not None
        if timed:
            start, end = _lib.time_next_launch(device)
        status = _lib.lib().ts_ema_multi(table.dev_ptr, table.n_chunks, table.chunk, float(m), 1.0 - float(m),
                                        _lib.current_stream_ptr(device))
        _lib.check(status, "ts_ema_multi")
        if timed:
            kernel_events.append((start, end))
        table.done()
    return views


class _Arena:
    """One flat output allocation and its views, shaped like a parameter list."""
    __slots__ = ("flat", "views", "ptrs", "numels", "stream", "readers", "__weakref__")

    def __init__(self, teachers: Sequence[torch.Tensor]):
        device = teachers[0].device
        # like a block of torch's caching allocator, the arena belongs to the
        # stream it was made on and is only handed out again on that stream
        self.stream = _lib.current_stream_ptr(device) if device.type == "cuda" else None
        numels = np.array(list(map(torch.Tensor.numel, teachers)), dtype=np.int64)
        dtype = teachers[0].dtype
        mask = 16 // teachers[0].element_size() - 1  # elements per 16 bytes, minus one
        if not (numels & mask).any():
            # every size is a multiple of 16 bytes: pieces sit back to back,
            # each on a 16-byte boundary, and torch's C++ unflatten makes the views
            self.flat = torch.empty(int(numels.sum()), dtype=dtype, device=device)
            self.views = list(torch._C._nn.unflatten_dense_tensors(self.flat, teachers))
        else:
            padded = ((numels + mask) & ~mask).tolist()
            self.flat = torch.empty(sum(padded), dtype=dtype, device=device)
            pieces = self.flat.split(padded)
            self.views = [p[:t.numel()].view(t.shape) for p, t in zip(pieces, teachers)]
        self.ptrs = _ptrs(self.views)
        self.numels = numels
        self.readers = []  # events of streams that read this version (note_reader)

    def is_free(self) -> bool:
        """True when nothing outside this arena can reach its memory: no view
        object is referenced elsewhere, from Python or from C++ (a tensor saved
        for a backward pass, a list kept by another extension), and the
        storage has no further alias."""
        storage = self.flat.untyped_storage()
        if _use_count(storage._cdata) != len(self.views) + 2:  # flat + views + the wrapper just made
            return False
        host = _lib.host_helper()
        if host is not None:
            return host.all_refcounts_equal(self.views, 1)  # only self.views holds them
        return all(c == 2 for c in map(sys.getrefcount, self.views)) and \
            all(c == 1 for c in map(torch.Tensor._use_count, self.views))


# Output arenas whose tensors the caller has dropped are handed out again
# (same tensor objects, same memory): making 150+ view tensors costs more host
# time than the kernel takes.  Keyed by (device, stream, shapes); a handful per key,
# matching the few parameter versions a pipeline keeps alive.
_POOL_LIMIT = 6
_pool = {}
_pool_lock = threading.Lock()
_recycle = True
_by_storage = {}  # data_ptr of an arena's flat allocation -> weak reference to the arena


def set_recycling(enabled: bool) -> None:
    """Switches the reuse of output arenas on (the default) or off.  With it
    off every call allocates a fresh flat buffer and fresh views, exactly as
    the reference's ``clone()`` does, at 100+ microseconds of host time per
    150-tensor list."""
    global _recycle
    _recycle = bool(enabled)
    if not _recycle:
        release_pool()


def note_reader(version: Sequence[torch.Tensor], stream: Optional["torch.cuda.Stream"] = None) -> None:
    """Tells the pool that ``stream`` (default: the current one) has work
    enqueued that reads ``version``, a list this module returned.  An event is
    recorded on that stream, and the arena is only written again after it.

    Needed when a version is read on a stream other than the one that made it
    and then dropped without a host synchronisation.  The reference's own
    reader, ``copy_model``, synchronises its copy stream before it returns
    (tspipe/gpu_task.py:718-724) and needs no note."""
    if not version:
        return
    first = version[0]
    ref = _by_storage.get(first.untyped_storage().data_ptr())
    arena = ref() if ref is not None else None
    if arena is None:
        return
    stream = stream if stream is not None else torch.cuda.current_stream(first.device)
    event = torch.cuda.Event()
    event.record(stream)
    with _pool_lock:
        arena.readers.append(event)


def release_pool() -> None:
    """Drops every cached output arena (memory returns to torch's allocator
    once the caller's own references are gone) and the cached chunk tables."""
    with _pool_lock:
        _pool.clear()
        _by_storage.clear()
    _tables.clear_table_cache()


def _acquire_arena(teachers: Sequence[torch.Tensor], shapes):
    """Returns (arena, views): an arena nobody else can reach and a fresh list
    of its view tensors.  The list is made while the pool lock is held, so a
    second thread asking for the same key sees the arena as taken.

    shapes: anything hashable that identifies the list's shapes (the tuple of
    shapes, or the helper's (count, total, 64-bit shape hash) triple)."""
    if _use_count is None or not _recycle:
        arena = _Arena(teachers)
        return arena, list(arena.views)
    device = teachers[0].device
    # (the raw handle: a torch Stream object per call costs more than the rest of this function)
    key = (device, _lib.current_stream_ptr(device), shapes)
    with _pool_lock:
        arenas = _pool.setdefault(key, [])
        for arena in arenas:
            if arena.is_free():
                # streams that were announced as readers of the old contents
                if arena.readers:
                    stream = torch.cuda.current_stream(device)
                    for event in arena.readers:
                        stream.wait_event(event)
                arena.readers = []
                return arena, list(arena.views)
        arena = _Arena(teachers)
        arenas.append(arena)
        _by_storage[arena.flat.untyped_storage().data_ptr()] = weakref.ref(arena)
        if len(arenas) > _POOL_LIMIT:
            old = arenas.pop(0)  # stays alive for as long as its user holds it
            _by_storage.pop(old.flat.untyped_storage().data_ptr(), None)
        return arena, list(arena.views)


@torch.no_grad()
def momentum_update(m: float, online_new_param: Iterable[Optional[torch.Tensor]],
                    target_param: Iterable[torch.Tensor], skip_none: bool = False) -> List[torch.Tensor]:
    """Returns new tensors ``t*m + s*(1-m)``; the inputs are left untouched.

    The results are views of one flat allocation.  "New" means not aliased by
    anything the caller still holds: tensors of an earlier result may be handed
    out again once the caller has dropped every reference to them."""
    fast = _fast_update(m, online_new_param, target_param)
    if fast is not None:
        return fast
    students, teachers, shapes = _prepare(online_new_param, target_param, skip_none)
    if not teachers:
        return []
    if teachers[0].dtype is not _F32:
        shapes = (shapes, teachers[0].dtype)  # arenas of another type are another pool entry
    arena, views = _acquire_arena(teachers, shapes)
    _launch(m, students, teachers, arena.ptrs, arena.numels)
    return views


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
    students, teachers, _ = _prepare(online_params, target_params, skip_none=False)
    if not teachers:
        return
    numels = np.array(list(map(torch.Tensor.numel, teachers)), dtype=np.int64)
    _launch(m, students, teachers, _ptrs(teachers), numels)
    for live, work in zip(target_params, teachers):
        if work.data_ptr() != live.data_ptr():  # a non-contiguous parameter was densified
            live.detach().copy_(work)


@torch.no_grad()
def clone_and_update(m: float, online_param: Iterable[torch.Tensor], target_param: Iterable[torch.Tensor]):
    """Fuses the pipeline's student clone with the EMA that follows it
    (tspipe/gpu_task.py:398 and 403-406): returns
    ``([p.detach().clone() for p in online_param], [t*m + p*(1-m) ...])`` from one
    kernel launch that reads every student and teacher value once."""
    students, teachers, shapes = _prepare(online_param, target_param, skip_none=False)
    if not teachers:
        return [], []
    if teachers[0].dtype is not _F32:
        raise TypeError("the fused clone + EMA launch is fp32 (use clone_params and momentum_update for other types)")
    ema_arena, views = _acquire_arena(teachers, shapes)  # views held: the second acquire cannot hand the same arena out
    clone_arena, clone_views = _acquire_arena(teachers, shapes)
    offset = clone_arena.flat.data_ptr() - ema_arena.flat.data_ptr()
    device = teachers[0].device
    with _lib.on_device(device):
        table = _tables.stage_ema(_ptrs(teachers), _ptrs(students), ema_arena.ptrs, ema_arena.numels, device)
        timed = kernel_events is not None
        if timed:
            start, end = _lib.time_next_launch(device)
        status = _lib.lib().ts_ema_clone_multi(table.dev_ptr, table.n_chunks, table.chunk, float(m), 1.0 - float(m),
                                              offset, _lib.current_stream_ptr(device))
        _lib.check(status, "ts_ema_clone_multi")
        if timed:
            kernel_events.append((start, end))
        table.done()
    return clone_views, views


# ---------------------------------------------------------------------------
# The EMA's neighbours in the optimizer step: whole-list clone and copy-in
# ---------------------------------------------------------------------------

def _check_copy_lists(srcs: Sequence[torch.Tensor], dsts: Sequence[torch.Tensor]) -> None:
    if len(srcs) != len(dsts):
        raise ValueError(f"list lengths differ: {len(srcs)} vs {len(dsts)}")
    for s, d in zip(srcs, dsts):
        if s.shape != d.shape or s.dtype != d.dtype:
            raise ValueError(f"copy needs matching shape and dtype: {tuple(s.shape)} {s.dtype} vs {tuple(d.shape)} {d.dtype}")
        if not (s.is_cuda and d.is_cuda) or s.device != d.device:
            raise TypeError("whole-list copies run on tensors of one GPU (no host fallback)")
        if not d.is_contiguous():
            raise ValueError("destination tensors must be contiguous")


@torch.no_grad()
def clone_params(params: Iterable[torch.Tensor]) -> List[torch.Tensor]:
    """``[p.detach().clone() for p in params]`` as one kernel launch: the copy
    of the student parameters the pipeline takes after every optimizer step
    (tspipe/gpu_task.py:398).  The clones are views of one flat allocation."""
    srcs = [p.detach() for p in params]
    if not srcs:
        return []
    if any(not s.is_cuda for s in srcs):
        raise TypeError("whole-list copies run on device tensors (no host fallback)")
    dense = [s if s.is_contiguous() else s.contiguous() for s in srcs]
    by_dtype = {}
    for i, s in enumerate(dense):
        by_dtype.setdefault(s.dtype, []).append(i)
    outs: List[Optional[torch.Tensor]] = [None] * len(dense)
    for dtype, idx in by_dtype.items():
        esize = dense[idx[0]].element_size()
        per16 = 16 // esize  # elements per 16 bytes: every clone starts on a 16-byte boundary
        padded = [(dense[i].numel() + per16 - 1) // per16 * per16 for i in idx]
        flat = torch.empty(sum(padded), dtype=dtype, device=dense[idx[0]].device)
        for i, piece in zip(idx, flat.split(padded)):
            outs[i] = piece[:dense[i].numel()].view(dense[i].shape)
    live = [(s, o) for s, o in zip(dense, outs) if s.numel()]
    with _lib.on_device(dense[0].device):
        _tables.copy_segments([s for s, _ in live], [o for _, o in live])
    return outs  # type: ignore[return-value]


@torch.no_grad()
def copy_params_(dst_params: Iterable[torch.Tensor], src_params: Iterable[torch.Tensor]) -> None:
    """``for p, new in zip(dst, src): p.copy_(new)`` as one kernel launch: how a
    stored parameter version reaches the live module (tspipe/gpu_task.py:706-724)."""
    dsts = [d.detach() for d in dst_params]
    srcs = [s.detach() for s in src_params]
    _check_copy_lists(srcs, dsts)
    srcs = [s if s.is_contiguous() else s.contiguous() for s in srcs]
    live = [(s, d) for s, d in zip(srcs, dsts) if s.numel()]
    if not live:
        return
    with _lib.on_device(dsts[0].device):
        _tables.copy_segments([s for s, _ in live], [d for _, d in live])


@torch.no_grad()
def bind_params_(params: Iterable[torch.Tensor], version: Iterable[torch.Tensor]) -> None:
    """Makes a stored parameter version the live one without moving a byte:
    every parameter is re-pointed at the version's tensor (``p.data = new``),
    where tspipe/gpu_task.py:721-723 copies it (``p.copy_(new)``, one launch per
    tensor).  The ``nn.Parameter`` objects, and so the module and any state
    keyed by them, stay the same.

    The live parameters then *alias* the stored version, so this is for
    parameters nobody updates in place: the momentum teacher, whose every new
    version is a fresh list from ``update_target_fn``.  The student's optimizer
    steps in place and needs ``copy_params_``."""
    ps, vs = list(params), list(version)
    if len(ps) != len(vs):
        raise ValueError(f"{len(ps)} parameters but {len(vs)} tensors in the version")
    for p, v in zip(ps, vs):
        if p.shape != v.shape or p.dtype != v.dtype or p.device != v.device:
            raise ValueError(f"version tensor {tuple(v.shape)}/{v.dtype}/{v.device} does not fit parameter "
                             f"{tuple(p.shape)}/{p.dtype}/{p.device}")
    for p, v in zip(ps, vs):
        p.data = v.detach()

