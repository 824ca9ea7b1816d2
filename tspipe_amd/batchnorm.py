"""DeferredBatchNorm on hand-written gfx950 kernels.

Same module as tspipe/batchnorm.py (class 17-120, converter 122-154): a
BatchNorm layer that normalises every micro-batch with that micro-batch's own
statistics but updates ``running_mean`` / ``running_var`` once per mini-batch,
from per-channel sums accumulated over ``chunks`` micro-batches.

What runs where:

* ``_track`` + the statistics pass of ``F.batch_norm(training=True)`` are one
  kernel pass over the input (``ts_bn_stats``): it adds the micro-batch's
  per-channel sum and sum of squares into the ``sum`` / ``sum_squares`` buffers
  and leaves the micro-batch mean and inverse standard deviation for the
  normalisation;
* ``_commit`` is ``ts_bn_commit`` (biased variance, the reference's rounding
  order, accumulators cleared on the device);
* the normalisation and its backward are ``ts_bn_apply`` / ``ts_bn_backward``.

State-dict keys, constructor arguments, the ``ValueError`` for inputs below 3-D
and the converter's sharing of parameters and running buffers are unchanged.
"""
from typing import Optional, TypeVar, cast

import numpy as np
import torch
from torch import Tensor, nn
from torch.nn.modules.batchnorm import _BatchNorm

from . import _lib

__all__ = ["DeferredBatchNorm"]

# the C++ autograd node of the optional host helper takes the training forward when it is there
# (tests switch it off to exercise the Python path)
_HOST_NODE = True

TModule = TypeVar("TModule", bound=nn.Module)


def _ptr(t: Optional[Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


class _LayerState:
    """Per-layer bookkeeping that changes on every call, kept off the module
    object itself: ``nn.Module.__setattr__`` is a slow path (several
    ``isinstance`` checks per assignment), and a forward used to take it four
    times."""

    __slots__ = ("counter", "tracked", "chunks", "_np", "shared")

    def __init__(self, chunks: int):
        self.counter = 0
        self.tracked = 0
        self.chunks = chunks
        # [0]: which half of the reduction workspace the next call uses; [1]: raw handle of the stream
        # whose kernels used the workspace last (0: none yet).  One piece of host memory seen as a numpy
        # array here and as a tensor by the C++ autograd node, which updates it from autograd's thread.
        self._np = np.zeros(2, dtype=np.int64)
        self.shared = torch.from_numpy(self._np)

    @property
    def parity(self) -> int:
        return int(self._np[0])

    @parity.setter
    def parity(self, v: int) -> None:
        self._np[0] = v

    @property
    def ws_stream(self):
        v = int(self._np[1])
        return v if v else None

    @ws_stream.setter
    def ws_stream(self, v) -> None:
        self._np[1] = v if v else 0

    def __deepcopy__(self, memo):
        new = _LayerState(self.chunks)
        new.counter, new.tracked = self.counter, self.tracked
        new._np[:] = self._np
        return new

    def __reduce__(self):
        return (_restore_state, (self.chunks, self.counter, self.tracked, int(self._np[0])))


def _restore_state(chunks, counter, tracked, parity):
    st = _LayerState(chunks)
    st.counter, st.tracked = counter, tracked
    st._np[0] = parity
    return st


def _dims(x: Tensor):
    n, c = int(x.shape[0]), int(x.shape[1])
    hw = x.numel() // (n * c) if n * c else 0
    return n, c, hw


def _require_fp32_cuda(x: Tensor) -> None:
    if not x.is_cuda:
        raise TypeError("DeferredBatchNorm kernels need a device tensor (no host fallback)")
    if x.dtype != torch.float32:
        raise TypeError(f"DeferredBatchNorm kernels are fp32 (got {x.dtype})")


class _NormalizeFn(torch.autograd.Function):
    """y = (x - mean) * invstd * weight + bias with the given per-channel
    statistics.  ``training``: the statistics are the micro-batch's own
    (``spread`` holds inverse standard deviations, and backward accounts for
    their dependence on x); otherwise they are the fixed running statistics
    (``spread`` holds variances, ``eps`` is added on the fly)."""

    @staticmethod
    def forward(ctx, x, weight, bias, mean, spread, layer: "DeferredBatchNorm", training: bool, eps: float):
        n, c, hw = _dims(x)
        y = torch.empty_like(x)
        with _lib.on_device(x.device):
            status = _lib.lib().ts_bn_apply(x.data_ptr(), y.data_ptr(), mean.data_ptr(), spread.data_ptr(),
                                            _ptr(weight), _ptr(bias), n, c, hw, 0 if training else 1, eps,
                                            _lib.current_stream_ptr(x.device))
        _lib.check(status, "ts_bn_apply")
        ctx.save_for_backward(x, weight, mean, spread)
        ctx.layer = layer
        ctx.training = training
        ctx.eps = eps
        ctx.has_bias = bias is not None
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, mean, spread = ctx.saved_tensors
        invstd = spread if ctx.training else torch.rsqrt(spread + ctx.eps)
        n, c, hw = _dims(x)
        dy = dy.contiguous()
        dx = torch.empty_like(x)
        dgb = torch.empty((2, c), dtype=torch.float32, device=x.device)
        dgamma, dbeta = dgb[0], dgb[1]
        layer = ctx.layer
        ws = layer._workspace(x)
        parity = layer._st.parity  # shared with the training forward: the calls of a layer alternate
        with _lib.on_device(x.device):
            status = _lib.lib().ts_bn_backward(x.data_ptr(), dy.data_ptr(), mean.data_ptr(), invstd.data_ptr(),
                                               _ptr(weight), dx.data_ptr(), dgamma.data_ptr(), dbeta.data_ptr(),
                                               ws.data_ptr() + 12 * c, parity, n, c, hw, 1 if ctx.training else 0,
                                               _lib.current_stream_ptr(x.device))
        layer._after_launch(status, parity, "ts_bn_backward")
        return (dx, dgamma if weight is not None else None, dbeta if ctx.has_bias else None,
                None, None, None, None, None)


class _TrainForwardFn(torch.autograd.Function):
    """Training forward of one micro-batch: statistics, their bookkeeping in
    the layer's accumulators and the normalisation in two launches
    (``ts_bn_forward_train``); backward as for ``_NormalizeFn``."""

    @staticmethod
    def forward(ctx, x, weight, bias, layer: "DeferredBatchNorm"):
        n, c, hw = _dims(x)
        y = torch.empty_like(x)
        stats = torch.empty((2, c), dtype=torch.float32, device=x.device)
        mean, invstd = stats[0], stats[1]
        ws = layer._workspace(x)
        parity = layer._st.parity
        with _lib.on_device(x.device):
            status = _lib.lib().ts_bn_forward_train(
                x.data_ptr(), y.data_ptr(), _ptr(weight), _ptr(bias), n, c, hw, layer.sum.data_ptr(),
                layer.sum_squares.data_ptr(), mean.data_ptr(), invstd.data_ptr(), ws.data_ptr() + 12 * c, parity,
                float(layer.eps), _lib.current_stream_ptr(x.device))
        layer._after_launch(status, parity, "ts_bn_forward_train")
        ctx.save_for_backward(x, weight, mean, invstd)
        ctx.layer = layer
        ctx.training = True
        ctx.eps = float(layer.eps)
        ctx.has_bias = bias is not None
        return y

    @staticmethod
    def backward(ctx, dy):
        return _NormalizeFn.backward(ctx, dy)[:3] + (None,)


class DeferredBatchNorm(_BatchNorm):
    """A BatchNorm layer that tracks several micro-batches before it updates
    its running statistics (tspipe/batchnorm.py:17-120)."""

    sum: Tensor
    sum_squares: Tensor

    def __init__(self, num_features: int, eps: float = 1e-5, momentum: Optional[float] = 0.1,
                 affine: bool = True, chunks: int = 1) -> None:
        super().__init__(num_features, eps, momentum, affine, track_running_stats=True)
        self.register_buffer("sum", torch.zeros_like(self.running_mean))
        self.register_buffer("sum_squares", torch.zeros_like(self.running_var))
        # reduction workspace of the kernels, not part of the state dict: 3C
        # floats that are zero between calls (stand-alone statistics: two sums
        # and a ticket counter per channel) and two halves of 2C floats that
        # the training forward and the backward alternate between
        # (``_parity`` says which one the next call reduces into)
        self.register_buffer("_ws", torch.zeros(7 * num_features), persistent=False)
        object.__setattr__(self, "_st", _LayerState(chunks))

    # the reference's public counters (tspipe/batchnorm.py:36-38), kept in the state object
    counter = property(lambda self: self._st.counter, lambda self, v: setattr(self._st, "counter", v))
    tracked = property(lambda self: self._st.tracked, lambda self, v: setattr(self._st, "tracked", v))
    chunks = property(lambda self: self._st.chunks, lambda self, v: setattr(self._st, "chunks", v))
    _parity = property(lambda self: self._st.parity, lambda self, v: setattr(self._st, "parity", v))

    def _check_input_dim(self, input: Tensor) -> None:
        if input.dim() <= 2:
            raise ValueError("expected at least 3D input (got %dD input)" % input.dim())

    def _require_state(self, x: Tensor) -> None:
        """The kernels read and write the accumulators, the running statistics
        and the affine parameters as C floats on x's device.  A module cast
        with ``.half()`` / ``.double()`` or left on another device is refused
        here, as ``F.batch_norm`` refuses mixed types, instead of letting a
        kernel write 4-byte values into narrower buffers."""
        dev, f32 = x.device, torch.float32
        bufs, params = self._buffers, self._parameters
        a, b, c, d = bufs["sum"], bufs["sum_squares"], bufs["running_mean"], bufs["running_var"]
        w, bias = params.get("weight"), params.get("bias")
        ok = (a.dtype is f32 and b.dtype is f32 and c.dtype is f32 and d.dtype is f32 and a.device == dev
              and b.device == dev and c.device == dev and d.device == dev
              and (w is None or (w.dtype is f32 and w.device == dev))
              and (bias is None or (bias.dtype is f32 and bias.device == dev)))
        nbt = bufs.get("num_batches_tracked")
        if ok and (nbt is None or (nbt.dtype is torch.int64 and nbt.device == dev)):
            return
        state = [("sum", a), ("sum_squares", b), ("running_mean", c), ("running_var", d), ("weight", w), ("bias", bias)]
        for name, t in state:
            if t is None:
                continue
            if t.dtype != torch.float32:
                raise TypeError(f"DeferredBatchNorm kernels are fp32: {name} is {t.dtype} (input {x.dtype})")
            if t.device != x.device:
                raise TypeError(f"DeferredBatchNorm: {name} is on {t.device}, the input on {x.device}")
        raise TypeError(f"DeferredBatchNorm: num_batches_tracked must be int64 on {x.device}")

    def _workspace(self, x: Tensor) -> Tensor:
        """The layer's reduction workspace, on x's device.  Its alternating
        halves assume that the layer's calls run one after the other on the
        device, so a call on a stream other than the previous call's first
        waits for that stream."""
        st = self._st
        ws = self._buffers["_ws"]
        if ws.device != x.device or ws.numel() != 7 * self.num_features or ws.dtype is not torch.float32:
            # moved, resized, or cast along with the module (module.half()): start from zeros
            ws = self._ws = torch.zeros(7 * self.num_features, dtype=torch.float32, device=x.device)
            st.parity = 0
            st.ws_stream = None
        stream = _lib.current_stream_ptr(x.device)
        if st.ws_stream is not None and st.ws_stream != stream:
            torch.cuda.current_stream(x.device).wait_stream(torch.cuda.ExternalStream(st.ws_stream, device=x.device))
        st.ws_stream = stream
        return ws

    def _after_launch(self, status: int, parity: int, what: str) -> None:
        """The half the next call reduces into alternates only once this call
        is known to have been enqueued.  A refused call may have run part of
        its launches, so the workspace starts again from zeros."""
        if status < 0:
            self._ws = torch.zeros(7 * self.num_features, dtype=torch.float32, device=self._ws.device)
            self._st.parity = 0
            _lib.check(status, what)
        self._st.parity = 1 - parity

    def _stats(self, x: Tensor, accumulate: bool):
        """One pass over x: micro-batch mean / invstd, optionally ``sum += ...``."""
        n, c, hw = _dims(x)
        mean = torch.empty(c, dtype=torch.float32, device=x.device)
        invstd = torch.empty(c, dtype=torch.float32, device=x.device)
        with _lib.on_device(x.device):
            status = _lib.lib().ts_bn_stats(
                x.data_ptr(), n, c, hw, self._workspace(x).data_ptr(),
                self.sum.data_ptr() if accumulate else None,
                self.sum_squares.data_ptr() if accumulate else None,
                mean.data_ptr(), invstd.data_ptr(), float(self.eps), _lib.current_stream_ptr(x.device))
        _lib.check(status, "ts_bn_stats")
        return mean, invstd

    def _track(self, input: Tensor) -> bool:
        """Adds a micro-batch to the accumulators (tspipe/batchnorm.py:45-59).
        Returns True once ``chunks`` micro-batches have been seen."""
        x = input.detach()
        _require_fp32_cuda(x)
        self._require_state(x)
        x = x if x.is_contiguous() else x.contiguous()
        self._last_stats = self._stats(x, accumulate=True)
        st = self._st
        st.counter += input.numel() // input.size(1)
        st.tracked += 1
        return st.tracked == st.chunks

    def _commit(self) -> None:
        """Folds the accumulated sums into the running statistics
        (tspipe/batchnorm.py:61-85)."""
        dev = self.sum.device
        if not self.sum.is_cuda:
            raise TypeError("DeferredBatchNorm kernels need device buffers (no host fallback)")
        self._require_state(self.sum)
        with _lib.on_device(dev):
            status = _lib.lib().ts_bn_commit(
                self.sum.data_ptr(), self.sum_squares.data_ptr(), self.running_mean.data_ptr(),
                self.running_var.data_ptr(), self.num_batches_tracked.data_ptr(), self.num_features,
                float(self.counter), -1.0 if self.momentum is None else float(self.momentum),
                _lib.current_stream_ptr(dev))
        _lib.check(status, "ts_bn_commit")
        self._st.counter = 0
        self._st.tracked = 0

    def forward(self, input: Tensor) -> Tensor:  # type: ignore[override]
        self._check_input_dim(input)
        _require_fp32_cuda(input)
        self._require_state(input)
        if input.size(1) != self.num_features:
            raise ValueError(f"expected {self.num_features} channels, got {input.size(1)}")
        x = input if input.is_contiguous() else input.contiguous()
        weight = self.weight if self.affine else None
        bias = self.bias if self.affine else None
        per_channel = input.numel() // input.size(1) if input.size(1) else 0
        if per_channel <= 1 and (self.training or per_channel == 0):
            return self._forward_without_a_batch(input, x, per_channel)

        if not self.training:
            # fixed running statistics (tspipe/batchnorm.py:88-99)
            if not (torch.is_grad_enabled() and (x.requires_grad or (weight is not None and weight.requires_grad)
                                                 or (bias is not None and bias.requires_grad))):
                # nothing to differentiate (a teacher network under no_grad): the launch alone
                n, c, hw = _dims(x)
                y = torch.empty_like(x)
                with _lib.on_device(x.device):
                    status = _lib.lib().ts_bn_apply(x.data_ptr(), y.data_ptr(), self.running_mean.data_ptr(),
                                                    self.running_var.data_ptr(), _ptr(weight), _ptr(bias), n, c, hw,
                                                    1, float(self.eps), _lib.current_stream_ptr(x.device))
                _lib.check(status, "ts_bn_apply")
                return y
            return _NormalizeFn.apply(x, weight, bias, self.running_mean, self.running_var,
                                      self, False, float(self.eps))

        # statistics of this micro-batch into the accumulators
        # (tspipe/batchnorm.py:45-59) and its normalisation (111-120), fused;
        # the commit (61-85) follows once ``chunks`` micro-batches are in
        st = self._st
        y = None
        host = _lib.host_helper()
        if host is not None and _HOST_NODE:
            # the same two launches and the same backward from a C++ autograd node (no interpreter in
            # backward); it shares the parity / last-stream words with this object
            ws = self._workspace(x)
            try:
                y = host.bn_train(x, weight, bias, self.sum, self.sum_squares, ws, st.shared, float(self.eps),
                                  st.ws_stream or 0)
            except RuntimeError:
                # a refused call may have run part of its launches: the workspace starts again from zeros
                self._ws = torch.zeros(7 * self.num_features, dtype=torch.float32, device=ws.device)
                st.parity = 0
                raise
        if y is None:
            y = _TrainForwardFn.apply(x, weight, bias, self)
        st.counter += input.numel() // input.size(1)
        st.tracked += 1
        if st.tracked == st.chunks:
            self._commit()
        return y

    def _forward_without_a_batch(self, input: Tensor, x: Tensor, per_channel: int) -> Tensor:
        """The two inputs no kernel normalises.  An empty micro-batch comes back
        empty; in training it still counts as tracked, and a commit over zero
        values leaves NaN running statistics (0/0), as tspipe/batchnorm.py:45-85
        does.  One value per channel in training is tracked and committed like
        any micro-batch (batchnorm.py:103-108) and then refused with the error
        that ``F.batch_norm(training=True)`` raises at batchnorm.py:111-120."""
        if self.training:
            if per_channel:
                self._stats(x.detach(), accumulate=True)
            st = self._st
            st.counter += per_channel
            st.tracked += 1
            if st.tracked == st.chunks:
                self._commit()
            if per_channel:
                raise ValueError(f"Expected more than 1 value per channel when training, got input size {input.size()}")
        return x.clone()

    @classmethod
    def convert_deferred_batch_norm(cls, module: TModule, chunks: int = 1) -> TModule:
        """Swaps every BatchNorm that tracks running statistics, at any depth,
        for a DeferredBatchNorm sharing its parameters and running buffers
        (tspipe/batchnorm.py:122-154)."""
        if isinstance(module, DeferredBatchNorm) and module.chunks is chunks:
            return cast(TModule, module)

        converted: nn.Module = module
        if isinstance(module, _BatchNorm) and module.track_running_stats:
            converted = DeferredBatchNorm(module.num_features, module.eps, module.momentum, module.affine, chunks)
            if module.affine:
                converted.register_parameter("weight", module.weight)
                converted.register_parameter("bias", module.bias)
            for name in ("running_mean", "running_var", "num_batches_tracked"):
                converted.register_buffer(name, getattr(module, name))
            if module.running_mean is not None and module.running_mean.device != converted.sum.device:
                dev = module.running_mean.device
                converted.sum = converted.sum.to(dev)
                converted.sum_squares = converted.sum_squares.to(dev)
                converted._ws = converted._ws.to(dev)

        for name, child in module.named_children():
            converted.add_module(name, cls.convert_deferred_batch_norm(child, chunks))
        return cast(TModule, converted)
