"""ctypes binding of libtspipe_amd.so (the C ABI declared in include/tspipe_amd.h).

The library is loaded lazily, once per process, so that the adapters can be
pickled into spawned worker processes the way TSPipe ships its plug-ins
(tspipe/gpu_worker.py:596-600).  There is no fallback: if the library is
missing, every operation raises.
"""
import ctypes
import os
import threading
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
# TSPIPE_AMD_LIBRARY names another build of the same C ABI (a measurement
# variant from `python -m tspipe_amd.build --variant NAME`); unset, the
# library next to this file is the one.
LIB_PATH = os.environ.get("TSPIPE_AMD_LIBRARY") or os.path.join(_HERE, "libtspipe_amd.so")

TS_F32, TS_BF16, TS_F16 = 0, 1, 2

_lock = threading.RLock()  # host_helper() loads lib() while holding it
_lib = None

# name -> (restype, argtypes); one row per symbol of include/tspipe_amd.h
SIGNATURES = {
    "ts_version": (c_char_p, []),
    "ts_error_string": (c_char_p, [c_int]),
    "ts_last_hip_error": (c_int, []),
    "ts_time_next_launch": (c_int, [c_void_p, c_void_p]),
    "ts_ema_auto_chunk": (c_int64, [c_int64]),
    "ts_ema_plan": (c_int64, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int64]),
    "ts_ema_multi": (c_int, [c_void_p, c_int64, c_int64, c_float, c_float, c_void_p]),
    "ts_ema_plan_dtype": (c_int64, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p,
                                    c_int64]),
    "ts_ema_multi_dtype": (c_int, [c_void_p, c_int64, c_int64, c_float, c_float, c_int, c_void_p]),
    "ts_ema_clone_multi": (c_int, [c_void_p, c_int64, c_int64, c_float, c_float, c_int64, c_void_p]),
    "ts_copy_auto_chunk": (c_int64, [c_int64]),
    "ts_copy_plan": (c_int64, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int64]),
    "ts_copy_segments": (c_int, [c_void_p, c_int64, c_int64, c_void_p]),
    "ts_kd_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int]),
    "ts_kd_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_float,
                              c_float, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "ts_kd_static_scratch_bytes": (c_size_t, []),
    "ts_kd_fwd_bwd_static": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_float,
                                     c_float, c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "ts_kdce_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                c_float, c_float, c_float, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "ts_kdce_pieces_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64,
                                       c_float, c_float, c_float, c_void_p, c_void_p, c_int, c_void_p]),
    "ts_cosine_workspace_bytes": (c_size_t, [c_int64]),
    "ts_cosine_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float, c_void_p, c_void_p,
                                  c_void_p, c_int, c_void_p]),
    "ts_cosine_pieces_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_float,
                                         c_void_p, c_void_p, c_int, c_void_p]),
    "ts_mse_pieces_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_float, c_int,
                                      c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "ts_mse_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "ts_mse_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_float, c_int, c_int,
                               c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "ts_scale_rows": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p]),
    "ts_byol_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p,
                                c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "ts_byol_pieces_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                       c_int64, c_void_p, c_void_p, c_int, c_void_p]),
    "ts_infonce_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int]),
    "ts_copy_few": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "ts_infonce_set_workgroup_target": (c_int, [c_int]),
    "ts_infonce_set_fp32_arithmetic": (c_int, [c_int]),
    "ts_infonce_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float,
                                   c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "ts_infonce_pieces_fwd_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                          c_int64, c_float, c_void_p, c_void_p, c_int, c_void_p]),
    "ts_bn_stats_workspace_bytes": (c_size_t, [c_int64]),
    "ts_bn_stats": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                            c_void_p, c_float, c_void_p]),
    "ts_bn_commit": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_double,
                             c_double, c_void_p]),
    "ts_bn_apply": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                            c_int64, c_int, c_float, c_void_p]),
    "ts_bn_forward_train": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                    c_void_p, c_void_p, c_void_p, c_int, c_float, c_void_p]),
    "ts_bn_backward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_void_p]),
}


class TSPipeAmdError(RuntimeError):
    """A C-ABI call returned a negative status."""


def lib() -> ctypes.CDLL:
    """Returns the loaded library, loading it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise ImportError(
                    f"{LIB_PATH} is missing: build it with `python -m tspipe_amd.build` "
                    "(hipcc, gfx950). There is no non-HIP fallback.")
            # torch brings its own libamdhip64.so.7; importing it first makes
            # this library bind to the same HIP runtime instance as torch's
            # allocator and streams.
            import torch  # noqa: F401
            handle = ctypes.CDLL(LIB_PATH)
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(handle, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = handle
    return _lib


HOST_LIB_PATH = os.path.join(_HERE, "_ts_hostlist.so")
_host = None
_host_tried = False


def host_helper():
    """The optional C++ list helper (tspipe_amd/csrc_host), or None when it has
    not been built.  It only walks Python lists of tensors faster; all GPU work
    goes through lib()."""
    global _host, _host_tried
    if _host_tried:
        return _host
    with _lock:
        if not _host_tried:
            if os.path.exists(HOST_LIB_PATH):
                import importlib.util
                import torch  # noqa: F401  (the module links against torch)
                spec = importlib.util.spec_from_file_location("_ts_hostlist", HOST_LIB_PATH)
                mod = importlib.util.module_from_spec(spec)
                spec.loader.exec_module(mod)
                if hasattr(mod, "bind_abi"):
                    handle = lib()
                    addr = lambda fn: ctypes.cast(fn, c_void_p).value  # noqa: E731
                    mod.bind_abi(addr(handle.ts_infonce_workspace_bytes), addr(handle.ts_infonce_fwd_bwd),
                                 addr(handle.ts_scale_rows))
                    if hasattr(mod, "bind_bn"):
                        mod.bind_bn(addr(handle.ts_bn_forward_train), addr(handle.ts_bn_backward))
                    if hasattr(mod, "bind_losses"):
                        mod.bind_losses(addr(handle.ts_kd_workspace_bytes), addr(handle.ts_kdce_fwd_bwd),
                                        addr(handle.ts_mse_workspace_bytes), addr(handle.ts_mse_fwd_bwd),
                                        addr(handle.ts_cosine_workspace_bytes), addr(handle.ts_cosine_fwd_bwd),
                                        addr(handle.ts_byol_fwd_bwd))
                _host = mod
            _host_tried = True
    return _host


def check(status: int, what: str) -> int:
    """Raises on a negative status; returns it otherwise (plans return counts)."""
    if status < 0:
        handle = lib()
        msg = handle.ts_error_string(int(status)).decode()
        hip = handle.ts_last_hip_error()
        raise TSPipeAmdError(f"{what}: {msg} (status {status}, last HIP error {hip})")
    return status


def dtype_code(dtype) -> int:
    import torch
    if dtype == torch.float32:
        return TS_F32
    if dtype == torch.bfloat16:
        return TS_BF16
    if dtype == torch.float16:
        return TS_F16
    raise TypeError(f"unsupported dtype {dtype}: the kernels take float32, bfloat16 or float16")


_event_pool = []


def prepare_timing_events(device, count: int) -> None:
    """Creates ``count`` pairs of timing events ahead of time, so that
    ``time_next_launch`` inside a timed region costs no event creation and no
    extra marker packet on the stream."""
    import torch
    stream = torch.cuda.current_stream(device)
    for _ in range(count):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        # a first record creates the HIP events; the launch re-records them
        start.record(stream)
        end.record(stream)
        _event_pool.append((start, end))


def time_next_launch(device):
    """Arms the calling thread so that the next EMA / copy kernel stamps its
    own begin and end into a pair of timing events (measurement aid); returns
    the pair for ``start.elapsed_time(end)`` after a synchronize."""
    if not _event_pool:
        prepare_timing_events(device, 1)
    start, end = _event_pool.pop()
    check(lib().ts_time_next_launch(start.cuda_event, end.cuda_event), "ts_time_next_launch")
    return start, end


class on_device:
    """``with torch.cuda.device(dev)`` only when `dev` is not already the
    current device: the context manager costs a training forward on a small
    feature map about as much host time as the rest of the call."""

    __slots__ = ("ctx",)

    def __init__(self, dev):
        self.ctx = None if dev.index == _torch().cuda.current_device() else _torch().cuda.device(dev)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


def _torch():
    import torch
    return torch


def current_stream_ptr(device) -> int:
    """Raw handle of torch's current stream on `device` (a torch.device or an
    index).  Through torch's C binding where it has one: building a Stream
    object costs the adapters more host time than some of the kernels take."""
    import torch
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None:
        index = device if isinstance(device, int) else device.index
        if index is None:
            index = torch.cuda.current_device()
        return raw(index)
    return torch.cuda.current_stream(device).cuda_stream
