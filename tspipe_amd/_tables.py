"""Chunk-table staging: host planner -> pinned buffer -> device buffer.

The EMA and multi-segment copy kernels walk a table of 32-byte entries in
device memory.  Tables are planned by the C library straight into pinned host
memory and copied with one asynchronous H2D transfer on the caller's stream.
A small ring of (pinned, device) buffer pairs per thread and device lets the
host run ahead of the GPU: a pair is reused only after the launch that last
read it has finished.
"""
import ctypes
import threading
from collections import OrderedDict
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


class CachedTable:
    """A table that stays on the device for as long as the cache keeps it."""
    __slots__ = ("dev", "n_chunks", "chunk", "key")

    def __init__(self, dev: torch.Tensor, n_chunks: int, chunk: int, key: bytes):
        self.dev, self.n_chunks, self.chunk, self.key = dev, n_chunks, chunk, key

    @property
    def dev_ptr(self) -> int:
        return self.dev.data_ptr()

    def done(self) -> None:
        pass


_TABLE_CACHE_ENTRIES = 8
# device index -> OrderedDict(key -> CachedTable); shared by all threads (the
# key names the stream, so threads on different streams never share an entry)
_table_caches = {}
_table_lock = threading.Lock()


def _table_cache(device: torch.device) -> "OrderedDict":
    key = device.index if device.index is not None else torch.cuda.current_device()
    cache = _table_caches.get(key)
    if cache is None:
        cache = _table_caches.setdefault(key, OrderedDict())
    return cache


def clear_table_cache() -> None:
    """Drops the cached device tables."""
    with _table_lock:
        _table_caches.clear()


def stage_ema(t_ptrs: np.ndarray, s_ptrs: np.ndarray, o_ptrs: np.ndarray, numels: np.ndarray,
              device: torch.device, chunk_elems: int = 0, dtype: int = 0):
    """Plans the chunk table of one EMA launch and puts it on the device.

    A training loop presents the same few (teacher, student, output) pointer
    lists over and over -- parameter versions rotate through a handful of
    buffers -- and the table is a pure function of those pointers.  So the last
    few tables stay resident, keyed by the pointer arrays themselves and the
    stream that uploaded them: a repeat costs neither the planning nor the
    host-to-device copy in front of the kernel."""
    lib = _lib.lib()
    n = len(numels)
    if chunk_elems == 0:
        chunk_elems = lib.ts_ema_auto_chunk(int(numels.sum()))
    stream_id = _lib.current_stream_ptr(device)
    key = b"".join((t_ptrs[:n].tobytes(), s_ptrs[:n].tobytes(), o_ptrs[:n].tobytes(), numels[:n].tobytes(),
                    int(chunk_elems).to_bytes(8, "little"), int(stream_id).to_bytes(8, "little"),
                    bytes((dtype,))))
    cache = _table_cache(device)
    with _table_lock:
        hit = cache.get(key)
        if hit is not None:
            cache.move_to_end(key)
            return hit
    args = (t_ptrs.ctypes.data, s_ptrs.ctypes.data, o_ptrs.ctypes.data, numels.ctypes.data, n, chunk_elems, dtype)
    ring = _ring(device)
    slot = ring.acquire(0)
    count = lib.ts_ema_plan_dtype(*args, slot.pinned.data_ptr(), slot.capacity)
    if count == -2:  # TS_ERR_CAPACITY: count, grow the slot, plan again
        count = _lib.check(lib.ts_ema_plan_dtype(*args, None, 0), "ts_ema_plan(count)")
        slot = ring.grow(slot, count)
        count = lib.ts_ema_plan_dtype(*args, slot.pinned.data_ptr(), slot.capacity)
    _lib.check(count, "ts_ema_plan")
    nbytes = count * ENTRY_BYTES
    dev = torch.empty(max(nbytes, ENTRY_BYTES), dtype=torch.uint8, device=device)
    if count:
        dev[:nbytes].copy_(slot.pinned[:nbytes], non_blocking=True)
    # the pinned half of the slot is free again once this copy has run
    StagedTable(slot, count, chunk_elems, device).done()
    entry = CachedTable(dev, count, chunk_elems, key)
    with _table_lock:
        cache[key] = entry
        while len(cache) > _TABLE_CACHE_ENTRIES:
            cache.popitem(last=False)
    return entry


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


FEW_SEGMENTS = 16            # what ts_copy_few takes
FEW_MAX_BYTES = 16 << 20     # longer segments go through the planned table (balanced chunks)


def copy_segments(srcs: Sequence[torch.Tensor], dsts: Sequence[torch.Tensor]) -> None:
    """dsts[i] <- srcs[i] (contiguous device tensors of equal byte size), one launch."""
    if not srcs:
        return
    copy_segments_raw([s.data_ptr() for s in srcs], [d.data_ptr() for d in dsts],
                      [s.numel() * s.element_size() for s in srcs], dsts[0].device)


def copy_segments_raw(src_ptrs: Sequence[int], dst_ptrs: Sequence[int], sizes: Sequence[int],
                      device: torch.device) -> None:
    """The same on device addresses and byte counts (the caller keeps the
    tensors alive until the launch is enqueued)."""
    n = len(src_ptrs)
    if n == 0:
        return
    if n <= FEW_SEGMENTS and kernel_events is None and max(sizes) <= FEW_MAX_BYTES:
        # a handful of small segments: described in the launch's own arguments, nothing planned or uploaded
        _lib.check(_lib.lib().ts_copy_few((ctypes.c_void_p * n)(*src_ptrs), (ctypes.c_void_p * n)(*dst_ptrs),
                                          (ctypes.c_int64 * n)(*sizes), n, _lib.current_stream_ptr(device)),
                   "ts_copy_few")
        return
    nbytes = np.asarray(sizes, dtype=np.int64)
    table = stage_copy(np.asarray(src_ptrs, dtype=np.uint64), np.asarray(dst_ptrs, dtype=np.uint64), nbytes, device)
    timed = kernel_events is not None
    if timed:
        start, end = _lib.time_next_launch(device)
    _lib.check(_lib.lib().ts_copy_segments(table.dev_ptr, table.n_chunks, table.chunk,
                                           _lib.current_stream_ptr(device)),
               "ts_copy_segments")
    if timed:
        kernel_events.append((start, end))
    table.done()
