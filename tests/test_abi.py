"""C-ABI checks that need no GPU: the library loads, exports every symbol the
header declares, rejects bad arguments before touching the device, and its
host-side planners produce correct chunk tables."""
import ctypes
import os
import re

import numpy as np
import pytest

from tspipe_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tspipe_amd.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ts_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.lib()
    names = declared_functions()
    assert len(names) >= 18
    for name in names:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names  # the ctypes table covers the header, no more, no less


def test_version_and_error_strings():
    lib = _lib.lib()
    assert b"tspipe_amd" in lib.ts_version()
    assert lib.ts_error_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5):
        assert lib.ts_error_string(code) not in (b"ok", b"unknown status")
    assert lib.ts_error_string(-99) == b"unknown status"
    with pytest.raises(_lib.TSPipeAmdError):
        _lib.check(-1, "demo")
    assert _lib.check(7, "count") == 7


class EmaChunk(ctypes.Structure):
    _fields_ = [("t", ctypes.c_uint64), ("s", ctypes.c_uint64), ("out", ctypes.c_uint64),
                ("n", ctypes.c_uint32), ("flags", ctypes.c_uint32)]


class CopyChunk(ctypes.Structure):
    _fields_ = [("src", ctypes.c_uint64), ("dst", ctypes.c_uint64), ("bytes", ctypes.c_uint64),
                ("flags", ctypes.c_uint64)]


def _u64(xs):
    return np.asarray(xs, dtype=np.uint64)


def _plan_ema(t, s, o, n, chunk, cap=None):
    lib = _lib.lib()
    t, s, o, n = _u64(t), _u64(s), _u64(o), np.asarray(n, dtype=np.int64)
    count = lib.ts_ema_plan(t.ctypes.data, s.ctypes.data, o.ctypes.data, n.ctypes.data, len(n), chunk, None, 0)
    if count < 0:
        return count, []
    cap = count if cap is None else cap
    table = (EmaChunk * max(cap, 1))()
    rc = lib.ts_ema_plan(t.ctypes.data, s.ctypes.data, o.ctypes.data, n.ctypes.data, len(n), chunk,
                         ctypes.addressof(table), cap)
    return rc, list(table)[:max(rc, 0)]


def test_ema_plan_covers_every_element_once():
    assert ctypes.sizeof(EmaChunk) == 32 and ctypes.sizeof(CopyChunk) == 32
    numels = [9408, 64, 0, 5000, 1, 2359296]
    base_t, base_s, base_o = 0x10000000, 0x20000000, 0x30000000
    offs = np.cumsum([0] + [((n + 3) & ~3) * 4 for n in numels[:-1]])
    t, s, o = base_t + offs, base_s + offs, base_o + offs
    rc, chunks = _plan_ema(t, s, o, numels, 4096)
    assert rc == sum((n + 4095) // 4096 for n in numels)
    covered = {i: 0 for i in range(len(numels))}
    for c in chunks:
        i = max(j for j in range(len(numels)) if numels[j] and t[j] <= c.t)
        off = (c.t - t[i]) // 4
        assert c.s - s[i] == c.t - t[i] == c.out - o[i]
        assert off % 4096 == 0 and c.n == min(4096, numels[i] - off)
        assert c.flags == 1
        covered[i] += c.n
    assert [covered[i] for i in range(len(numels))] == numels


def test_ema_plan_alignment_flags_and_errors():
    lib = _lib.lib()
    rc, chunks = _plan_ema([0x1000, 0x2004, 0x3000], [0x5000, 0x6004, 0x7008], [0x9000, 0xa004, 0xb000], [8, 8, 8], 4096)
    assert rc == 3 and [c.flags for c in chunks] == [1, 0, 0]
    assert _plan_ema([0x1002], [0x2000], [0x3000], [8], 4096)[0] == -4      # not 4-byte aligned
    assert _plan_ema([0x1000], [0x2000], [0x3000], [8], 1000)[0] == -1      # chunk not a multiple of 1024
    assert _plan_ema([0x1000], [0x2000], [0x3000], [-1], 4096)[0] == -1
    assert _plan_ema([0], [0x2000], [0x3000], [8], 4096)[0] == -1           # null tensor pointer
    assert _plan_ema([0x1000], [0x2000], [0x3000], [10000], 4096, cap=2)[0] == -2
    assert _plan_ema([], [], [], [], 0)[0] == 0
    # auto chunk: a multiple of 4096 that keeps the table near 4096 entries
    for total in (1, 4096, 11_689_512, 86_567_656, 10 ** 10):
        c = lib.ts_ema_auto_chunk(total)
        assert c % 4096 == 0 and c >= 4096 and (total + c - 1) // c <= 4096 + 1
    rc, chunks = _plan_ema([0x1000], [0x200000], [0x400000], [100000], 0)
    assert rc == (100000 + 4095) // 4096


def test_ema_plan_for_two_byte_types():
    lib = _lib.lib()
    numels = [5000, 3, 4096]
    t, s, o = _u64([0x10000, 0x20002, 0x30000]), _u64([0x50000, 0x60002, 0x70000]), _u64([0x90000, 0xa0002, 0xb0000])
    n = np.asarray(numels, dtype=np.int64)
    for dtype in (1, 2):  # TS_BF16, TS_F16
        args = (t.ctypes.data, s.ctypes.data, o.ctypes.data, n.ctypes.data, 3, 2048, dtype)
        count = lib.ts_ema_plan_dtype(*args, None, 0)
        assert count == 3 + 1 + 2
        table = (EmaChunk * count)()
        assert lib.ts_ema_plan_dtype(*args, ctypes.addressof(table), count) == count
        # element pointers advance by 2 bytes per element; the 2-byte aligned tensor is flagged
        assert [(c.t - 0x10000, c.n) for c in table[:3]] == [(0, 2048), (4096, 2048), (8192, 904)]
        assert table[3].t == 0x20002 and table[3].n == 3 and table[3].flags == 0
        assert [c.flags for c in table[:3]] == [1, 1, 1] and table[5].out == 0xb0000 + 4096
    bad = (t.ctypes.data, s.ctypes.data, o.ctypes.data, n.ctypes.data, 3)
    assert lib.ts_ema_plan_dtype(*bad, 1024, 1, None, 0) == -1   # 2-byte chunks are multiples of 2048
    assert lib.ts_ema_plan_dtype(*bad, 2048, 7, None, 0) == -1   # unknown dtype
    odd = _u64([0x10001])
    assert lib.ts_ema_plan_dtype(odd.ctypes.data, s.ctypes.data, o.ctypes.data, n.ctypes.data, 1, 2048, 1, None, 0) == -4
    # dtype 0 is ts_ema_plan itself
    assert lib.ts_ema_plan_dtype(*bad, 4096, 0, None, 0) == lib.ts_ema_plan(*bad, 4096, None, 0)


def _plan_copy(src, dst, nbytes, chunk, cap=None):
    lib = _lib.lib()
    src, dst, nbytes = _u64(src), _u64(dst), np.asarray(nbytes, dtype=np.int64)
    count = lib.ts_copy_plan(src.ctypes.data, dst.ctypes.data, nbytes.ctypes.data, len(nbytes), chunk, None, 0)
    if count < 0:
        return count, []
    cap = count if cap is None else cap
    table = (CopyChunk * max(cap, 1))()
    rc = lib.ts_copy_plan(src.ctypes.data, dst.ctypes.data, nbytes.ctypes.data, len(nbytes), chunk,
                          ctypes.addressof(table), cap)
    return rc, list(table)[:max(rc, 0)]


def test_copy_plan():
    rc, chunks = _plan_copy([0x1000, 0x9003, 0x20000], [0x100000, 0x200000, 0x300010], [40000, 7, 0], 16384)
    assert rc == 4
    assert [c.bytes for c in chunks] == [16384, 16384, 7232, 7]
    assert [c.flags for c in chunks] == [1, 1, 1, 0]
    assert chunks[1].src == 0x1000 + 16384 and chunks[1].dst == 0x100000 + 16384
    assert _plan_copy([0x1000], [0x2000], [10], 100)[0] == -1
    assert _plan_copy([0x1000], [0], [10], 16384)[0] == -1
    assert _plan_copy([0x1000], [0x2000], [100000], 16384, cap=1)[0] == -2
    lib = _lib.lib()
    for total in (1, 500_072_448, 10 ** 11):
        c = lib.ts_copy_auto_chunk(total)
        assert c % 16384 == 0 and (total + c - 1) // c <= 4096 + 1


def test_device_entry_points_validate_before_launching():
    """Argument errors are reported without any HIP call (so this runs on a CPU-only host)."""
    lib = _lib.lib()
    p = 0x1000
    assert lib.ts_ema_multi(None, 5, 4096, 0.9, 0.1, None) == -1
    assert lib.ts_ema_multi(p, -1, 4096, 0.9, 0.1, None) == -1
    assert lib.ts_ema_multi(p, 5, 1000, 0.9, 0.1, None) == -1
    assert lib.ts_ema_multi(p, 0, 4096, 0.9, 0.1, None) == 0           # nothing to do
    # a grid dimension times the workgroup size (256) must stay below 2^32 threads: the chunk count above
    # 65535 runs as a flat grid of chunks x sub-blocks
    assert lib.ts_ema_multi(p, 70000, 1024 * 300, 0.9, 0.1, None) == -5
    assert lib.ts_ema_multi(p, 1, 1024 * (1 << 24), 0.9, 0.1, None) == -5
    assert lib.ts_copy_segments(p, 1 << 25, 4096, None) == -5
    assert lib.ts_copy_segments(None, 3, 16384, None) == -1
    import ctypes
    three = (ctypes.c_void_p * 3)(p, p, p)
    assert lib.ts_copy_few(three, three, (ctypes.c_int64 * 3)(1, 2, 3), 17, None) == -5   # the table form takes more
    assert lib.ts_copy_few(None, three, (ctypes.c_int64 * 3)(1, 2, 3), 3, None) == -1
    assert lib.ts_copy_few(three, three, (ctypes.c_int64 * 3)(1, -2, 3), 3, None) == -1
    assert lib.ts_copy_few(three, three, (ctypes.c_int64 * 3)(0, 0, 0), 3, None) == 0        # nothing to copy
    assert lib.ts_copy_few(None, None, None, 0, None) == 0
    assert lib.ts_copy_segments(p, 0, 16384, None) == 0
    assert lib.ts_kd_fwd_bwd(None, p, None, 4, 10, 10, 10, 1.0, 1.0, p, p, None, 10, 0, None) == -1
    assert lib.ts_kd_fwd_bwd(p, p, None, 4, 10, 9, 10, 1.0, 1.0, p, p, None, 10, 0, None) == -1   # ld < V
    assert lib.ts_kd_fwd_bwd(p, p, None, 4, 10, 10, 10, 1.0, 1.0, p, p, None, 10, 7, None) == -1  # dtype
    assert lib.ts_kd_fwd_bwd(p + 1, p, None, 4, 10, 10, 10, 1.0, 1.0, p, p, None, 10, 0, None) == -4
    assert lib.ts_kd_fwd_bwd(p, p, None, 1 << 25, 10, 10, 10, 1.0, 1.0, p, p, None, 10, 0, None) == -5
    assert lib.ts_byol_fwd_bwd(p, p, p, None, 4, 8, p, p, None, None, 0, None) == -1              # x2 without y2
    assert lib.ts_infonce_fwd_bwd(p, p, None, None, 16, 600, 0.2, 0x1000, p, None, None, 1, None) == -5  # wider than 512
    assert lib.ts_infonce_fwd_bwd(p, p, None, None, 16, 64, 0.0, 0x1000, p, None, None, 1, None) == -1   # temperature
    assert lib.ts_infonce_fwd_bwd(p, p, None, None, 16, 64, 0.2, 0x1010, p, None, None, 1, None) == -4   # workspace alignment
    assert lib.ts_infonce_fwd_bwd(p, p, None, None, 16, 64, 0.2, 0x1000, p, None, None, 7, None) == -1   # dtype
    # the scheduling knob: returns the previous value; out-of-range values restore the default; the workspace
    # size does not follow it
    ws_bytes = lib.ts_infonce_workspace_bytes(4096, 256, 1)
    assert lib.ts_infonce_set_workgroup_target(32) == 256
    assert lib.ts_infonce_workspace_bytes(4096, 256, 1) == ws_bytes
    assert lib.ts_infonce_set_workgroup_target(100000) == 32
    assert lib.ts_infonce_set_workgroup_target(-3) == 256
    assert lib.ts_infonce_set_workgroup_target(0) == 256
    # the accuracy switch: returns the previous setting, leaves the workspace size alone
    assert lib.ts_infonce_set_fp32_arithmetic(1) == 0
    assert lib.ts_infonce_workspace_bytes(4096, 256, 1) == ws_bytes
    assert lib.ts_infonce_set_fp32_arithmetic(0) == 1
    assert lib.ts_infonce_set_fp32_arithmetic(0) == 0
    assert lib.ts_bn_stats(None, 2, 3, 4, p, None, None, None, None, 1e-5, None) == -1
    assert lib.ts_bn_stats(p, 2, 70000, 4, p, None, None, None, None, 1e-5, None) == -5
    assert lib.ts_bn_stats(p, 2, 3, 4, p, p, None, None, None, 1e-5, None) == -1                 # sum without sum_squares
    assert lib.ts_bn_commit(p, p, p, p, None, 8, 100.0, -1.0, None) == -1                        # momentum=None needs the counter
    assert lib.ts_bn_apply(p, None, p, p, None, None, 2, 3, 4, 0, 1e-5, None) == -1
    assert lib.ts_bn_backward(p, p, p, p, None, p, p, None, p, 0, 2, 3, 4, 1, None) == -1
    assert lib.ts_bn_backward(p, p, p, p, None, p, p, p, p, 2, 2, 3, 4, 1, None) == -1   # parity
    assert lib.ts_scale_rows(p, 4, 10, 9, p, 0, None) == -1
    assert lib.ts_kd_workspace_bytes(0, 100, 0) == 32 and lib.ts_kd_workspace_bytes(5, 100, 0) == 32 + 3 * 32
    assert lib.ts_kd_workspace_bytes(4096, 30522, 1) == 32 + 3 * 4096 * 4 + 4096 * 4 * 32  # 4 parts per wide row
    assert lib.ts_kdce_fwd_bwd(p, p, None, p + 4, -100, 4, 10, 10, 10, 1.0, 1.0, 1.0, p, p, None, 10, 0, None) == -4  # labels not 8-byte aligned
    assert lib.ts_kdce_fwd_bwd(p, p, None, None, -100, 4, 10, 10, 10, 0.0, 1.0, 1.0, p, p, None, 10, 0, None) == -1    # inv_T must be positive
    assert lib.ts_cosine_fwd_bwd(p, None, None, 4, 8, 1.0, p, p, None, 0, None) == -1
    assert lib.ts_cosine_workspace_bytes(5) == 48
    assert lib.ts_infonce_workspace_bytes(4096, 256, 1) > 4096 * 256 * 4
    assert lib.ts_infonce_workspace_bytes(4096, 256, 3) == 0


def test_measurement_variants_name_macros_their_sources_use():
    # `python -m tspipe_amd.build --variant NAME` rebuilds one source under macros: each macro must
    # exist in that source, or the variant would silently equal the default build
    from tspipe_amd import build
    for name, (src, defines) in build.VARIANTS.items():
        text = open(os.path.join(build.CSRC, src)).read()
        assert src in build.SOURCES, name
        for d in defines:
            assert f"#ifdef {d}" in text, (name, d)
