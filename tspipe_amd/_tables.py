"""Chunk-table staging: host planner -> pinned buffer -> device buffer.

The EMA and multi-segment copy kernels walk a table of 32-byte entries in
device memory.  Tables are planned by the C library straight into pinned host
memory and copied with one asynchronous H2D transfer on the caller's stream.
A small ring of (pinned, device) buffer pairs per thread and device lets the
host run ahead of the GPU: a pair is reused only after the launch that last
read it has finished.
"""
import threading
from typing import List, Sequence

import numpy as np
import torch

from . import _lib

ENTRY_BYTES = 32
_RING = 4
# When set to a list, every multi-segment copy appends a (start, end) pair of
# HIP events stamped with the kernel's own begin and end (profiling aid).
kernel_events = None
_tls = threading.local()


class _Slot:
    __slots__ = ("pinned", "dev", "event", "spare", "capacity")

    def __init__(self, device: torch.device, capacity: int):
        self.capacity = capacity
        self.spare = None  # the event object of the previous use, recycled
        self.pinned = torch.empty(capacity * ENTRY_BYTES, dtype=torch.uint8, pin_memory=True)
        self.dev = torch.empty(capacity * ENTRY_BYTES, dtype=torch.uint8, device=device)
        self.event = None


class _Ring:
    def __init__(self, device: torch.device):
        self.device = device
        self.slots: List[_Slot] = []
        self.next = 0

    def acquire(self, n_entries: int) -> _Slot:
        if len(self.slots) < _RING:
            slot = _Slot(self.device, max(n_entries, 4608))
            self.slots.append(slot)
            return slot
        idx = self.next
        self.next = (self.next + 1) % _RING
        slot = self.slots[idx]
        if slot.event is not None:
            slot.event.synchronize()  # the launch that read this table is done
            slot.spare, slot.event = slot.event, None
        if slot.capacity < n_entries:
            slot = self.grow(slot, n_entries)
        return slot

    def grow(self, slot: _Slot, n_entries: int) -> _Slot:
        """Replaces an idle slot by a larger one."""
        bigger = _Slot(self.device, max(n_entries, 2 * slot.capacity))
        self.slots[self.slots.index(slot)] = bigger
        return bigger


def _ring(device: torch.device) -> _Ring:
    rings = getattr(_tls, "rings", None)
    if rings is None:
        rings = _tls.rings = {}
    key = device.index if device.index is not None else torch.cuda.current_device()
    ring = rings.get(key)
    if ring is None:
        ring = rings[key] = _Ring(torch.device("cuda", key))
    return ring


def ptr_array(tensors: Sequence[torch.Tensor]) -> np.ndarray:
    return np.fromiter((t.data_ptr() for t in tensors), dtype=np.uint64, count=len(tensors))


class StagedTable:
    """A planned table resident on the device; call done() after the launch."""
    __slots__ = ("slot", "n_chunks", "chunk", "device")

    def __init__(self, slot: _Slot, n_chunks: int, chunk: int, device: torch.device):
        self.slot, self.n_chunks, self.chunk, self.device = slot, n_chunks, chunk, device

    @property
    def dev_ptr(self) -> int:
        return self.slot.dev.data_ptr()

    def done(self) -> None:
        ev = self.slot.spare or torch.cuda.Event()
        ev.record(torch.cuda.current_stream(self.device))
        self.slot.event = ev


def stage_ema(t_ptrs: np.ndarray, s_ptrs: np.ndarray, o_ptrs: np.ndarray, numels: np.ndarray,
              device: torch.device, chunk_elems: int = 0) -> StagedTable:
    lib = _lib.lib()
    n = len(numels)
    if chunk_elems == 0:
        chunk_elems = lib.ts_ema_auto_chunk(int(numels.sum()))
    args = (t_ptrs.ctypes.data, s_ptrs.ctypes.data, o_ptrs.ctypes.data, numels.ctypes.data, n, chunk_elems)
    ring = _ring(device)
    slot = ring.acquire(0)
    count = lib.ts_ema_plan(*args, slot.pinned.data_ptr(), slot.capacity)
    if count == -2:  # TS_ERR_CAPACITY: count, grow the slot, plan again
        count = _lib.check(lib.ts_ema_plan(*args, None, 0), "ts_ema_plan(count)")
        slot = ring.grow(slot, count)
        count = lib.ts_ema_plan(*args, slot.pinned.data_ptr(), slot.capacity)
    _lib.check(count, "ts_ema_plan")
    if count:
        nbytes = count * ENTRY_BYTES
        slot.dev[:nbytes].copy_(slot.pinned[:nbytes], non_blocking=True)
    return StagedTable(slot, count, chunk_elems, device)


def stage_copy(src_ptrs: np.ndarray, dst_ptrs: np.ndarray, nbytes_arr: np.ndarray,
               device: torch.device, chunk_bytes: int = 0) -> StagedTable:
    lib = _lib.lib()
    n = len(nbytes_arr)
    if chunk_bytes == 0:
        chunk_bytes = lib.ts_copy_auto_chunk(int(nbytes_arr.sum()))
    args = (src_ptrs.ctypes.data, dst_ptrs.ctypes.data, nbytes_arr.ctypes.data, n, chunk_bytes)
    ring = _ring(device)
    slot = ring.acquire(0)
    count = lib.ts_copy_plan(*args, slot.pinned.data_ptr(), slot.capacity)
    if count == -2:  # TS_ERR_CAPACITY: count, grow the slot, plan again
        count = _lib.check(lib.ts_copy_plan(*args, None, 0), "ts_copy_plan(count)")
        slot = ring.grow(slot, count)
        count = lib.ts_copy_plan(*args, slot.pinned.data_ptr(), slot.capacity)
    _lib.check(count, "ts_copy_plan")
    if count:
        nbytes = count * ENTRY_BYTES
        slot.dev[:nbytes].copy_(slot.pinned[:nbytes], non_blocking=True)
    return StagedTable(slot, count, chunk_bytes, device)


def copy_segments(srcs: Sequence[torch.Tensor], dsts: Sequence[torch.Tensor]) -> None:
    """dsts[i] <- srcs[i] (contiguous device tensors of equal byte size), one launch."""
    if not srcs:
        return
    device = dsts[0].device
    nbytes = np.fromiter((s.numel() * s.element_size() for s in srcs), dtype=np.int64, count=len(srcs))
    table = stage_copy(ptr_array(srcs), ptr_array(dsts), nbytes, device)
    timed = kernel_events is not None
    if timed:
        start, end = _lib.time_next_launch(device)
    _lib.check(_lib.lib().ts_copy_segments(table.dev_ptr, table.n_chunks, table.chunk,
                                           _lib.current_stream_ptr(device)),
               "ts_copy_segments")
    if timed:
        kernel_events.append((start, end))
    table.done()
