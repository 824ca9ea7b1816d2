"""Teacher-student losses with fused forward+backward HIP kernels, behind the
``loss_fn`` plug-in signatures TSPipe calls (tspipe/gpu_task.py:178-179 for
distillation, 202-203 for self-supervised momentum training).

Each loss is a ``torch.autograd.Function`` whose forward launches one fused
kernel that produces the scalar loss *and* the gradient with respect to the
student input; backward hands that gradient out (rescaled on the device by the
incoming gradient, which is exactly 1 when the pipeline calls
``torch.autograd.backward(loss)``, tspipe/gpu_task.py:207-212).  Teacher inputs
receive no gradient: the pipeline detaches them (tspipe/gpu_task.py:109).

The scalar loss is returned in fp32 whatever the input dtype, since the
kernels accumulate in fp32.
"""
from argparse import Namespace
from typing import Optional

import torch
from torch import Tensor, nn

from . import _lib


def _require_cuda(*tensors: Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise TypeError("tspipe_amd losses run on device tensors only (no host fallback)")


def _once(ctx) -> None:
    if ctx.backward_done:
        raise RuntimeError("the fused loss keeps one gradient buffer: backward can run once per forward")
    ctx.backward_done = True


def _scale_saved_grad(grad: Tensor, grad_output: Tensor, rows: int, cols: int) -> Tensor:
    """grad *= grad_output on the device, without a host sync; the kernel
    returns immediately when grad_output is 1."""
    g = grad_output.detach().to(torch.float32).reshape(1)
    with _lib.on_device(grad.device):
        status = _lib.lib().ts_scale_rows(grad.data_ptr(), rows, cols, cols, g.data_ptr(),
                                          _lib.dtype_code(grad.dtype), _lib.current_stream_ptr(grad.device))
    _lib.check(status, "ts_scale_rows")
    return grad


_HOST_NODE = True   # tests switch this off to reach the Python autograd.Functions
_KD, _MSE, _COSINE, _BYOL = 0, 1, 2, 3


def _host_row_loss(kind: int, x1, y1, x2, y2, mask, labels, f, n):
    """The plain case of a row loss through the C++ autograd node of the host
    helper (the same entry points in the same order as the Python Functions
    below, so the same bits; its backward needs no interpreter).  None when the
    helper is not built or the call is not plain: then the Python Function takes
    it, and raises the proper errors."""
    if not _HOST_NODE:
        return None
    host = _lib.host_helper()
    if host is None or type(x1) is not Tensor or not x1.is_cuda or not hasattr(host, "row_loss"):
        return None
    return host.row_loss(kind, x1, y1, x2, y2, mask, labels, f, n, _lib.current_stream_ptr(x1.device))


# ---------------------------------------------------------------------------
# KD soft-target loss
# ---------------------------------------------------------------------------

class _KDSoftTargetFn(torch.autograd.Function):
    """KD soft-target term, optionally with the hard-label CE term, in one pass
    over the student logits; optionally followed by the logits-MSE term over
    the same rows, added in place to the loss and to the gradient."""

    @staticmethod
    def forward(ctx, out_s: Tensor, out_t: Tensor, row_mask: Optional[Tensor], T: float, weight: float,
                labels: Optional[Tensor] = None, ce_weight: float = 0.0, ignore_index: int = -100,
                mse_weight: float = 0.0, mse_per_element: bool = False):
        _require_cuda(out_s, out_t, row_mask, labels)
        if out_s.shape != out_t.shape:
            raise ValueError(f"student/teacher logits differ in shape: {tuple(out_s.shape)} vs {tuple(out_t.shape)}")
        if out_s.dtype != out_t.dtype:
            raise TypeError(f"student/teacher logits differ in dtype: {out_s.dtype} vs {out_t.dtype}")
        V = int(out_s.shape[-1])
        s = out_s.detach().reshape(-1, V)
        t = out_t.detach().reshape(-1, V)
        s = s if s.is_contiguous() else s.contiguous()
        t = t if t.is_contiguous() else t.contiguous()
        rows = int(s.shape[0])
        mask_ptr = None
        if row_mask is not None:
            m = row_mask.detach().reshape(-1)
            if m.numel() != rows:
                raise ValueError(f"row mask has {m.numel()} entries for {rows} rows")
            if m.dtype != torch.bool:
                m = m != 0
            m = m.contiguous().view(torch.uint8)
            mask_ptr = m.data_ptr()
        label_ptr = None
        if labels is not None:
            lab = labels.detach().reshape(-1)
            if lab.numel() != rows:
                raise ValueError(f"{lab.numel()} labels for {rows} rows")
            if lab.dtype != torch.int64:
                lab = lab.to(torch.int64)
            lab = lab.contiguous()
            label_ptr = lab.data_ptr()
        need_grad = ctx.needs_input_grad[0]
        lib = _lib.lib()
        dev = s.device
        code = _lib.dtype_code(s.dtype)
        ws = torch.empty(lib.ts_kd_workspace_bytes(rows, V, code), dtype=torch.uint8, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        grad = torch.empty_like(s) if need_grad else None
        with _lib.on_device(dev):
            status = lib.ts_kdce_fwd_bwd(s.data_ptr(), t.data_ptr(), mask_ptr, label_ptr, int(ignore_index), rows, V,
                                         V, V, 1.0 / T, T * T * weight, float(ce_weight), ws.data_ptr(),
                                         loss.data_ptr(), None if grad is None else grad.data_ptr(), V, code,
                                         _lib.current_stream_ptr(dev))
        _lib.check(status, "ts_kdce_fwd_bwd")
        if mse_weight > 0.0:
            ws2 = torch.empty(lib.ts_mse_workspace_bytes(rows, V), dtype=torch.uint8, device=dev)
            with _lib.on_device(dev):
                status = lib.ts_mse_fwd_bwd(s.data_ptr(), t.data_ptr(), mask_ptr, rows, V, V, V, float(mse_weight),
                                            1 if mse_per_element else 0, 1,
                                            ws2.data_ptr(), loss.data_ptr(), None if grad is None else grad.data_ptr(),
                                            V, code, _lib.current_stream_ptr(dev))
            _lib.check(status, "ts_mse_fwd_bwd")
        ctx.grad = grad
        ctx.shape = out_s.shape
        ctx.dims = (rows, V)
        ctx.backward_done = False
        return loss

    @staticmethod
    def backward(ctx, grad_output: Tensor):
        if ctx.grad is None:
            return (None,) * 10
        _once(ctx)
        grad = _scale_saved_grad(ctx.grad, grad_output, *ctx.dims)
        return (grad.view(ctx.shape),) + (None,) * 9


def kd_soft_target_loss(out_s: Tensor, out_t: Tensor, T: float, weight: float = 1.0,
                        row_mask: Optional[Tensor] = None) -> Tensor:
    """``weight * T^2 * KL(softmax(out_t/T) || softmax(out_s/T))`` averaged over
    the rows (last dimension = classes) selected by ``row_mask`` (all rows when
    ``None``); the formula of benchmarks/soft_target/kd_losses/st.py:18-23 and,
    with a mask, of benchmarks/distilbert/distiller.py:719-740."""
    out = _host_row_loss(_KD, out_s, out_t, None, None, row_mask, None, [float(T), float(weight), 0.0, 0.0], [-100, 0])
    if out is not None:
        return out
    return _KDSoftTargetFn.apply(out_s, out_t, row_mask, float(T), float(weight))


class SoftTarget(nn.Module):
    """Drop-in for benchmarks/soft_target/kd_losses/st.py:9-23."""

    def __init__(self, T: float):
        super().__init__()
        self.T = T

    def forward(self, out_s: Tensor, out_t: Tensor) -> Tensor:
        if out_s.dim() != 2:
            raise ValueError("SoftTarget expects [batch, classes] logits")
        return kd_soft_target_loss(out_s, out_t, self.T)


def distil_ce_loss(s_logits: Tensor, t_logits: Tensor, row_mask: Tensor, temperature: float,
                   alpha_ce: float = 1.0) -> Tensor:
    """The distillation term of DistilBERT's loss
    (benchmarks/distilbert/distiller.py:719-740): rows of ``[bs, seq, vocab]``
    logits where ``row_mask`` (``[bs, seq]``) is set, KL with batchmean over the
    selected rows, times ``temperature**2`` and ``alpha_ce``.  No row is copied:
    the kernel reads the mask and writes a dense gradient with zeros elsewhere."""
    out = _host_row_loss(_KD, s_logits, t_logits, None, None, row_mask, None,
                         [float(temperature), float(alpha_ce), 0.0, 0.0], [-100, 0])
    if out is not None:
        return out
    return _KDSoftTargetFn.apply(s_logits, t_logits, row_mask, float(temperature), float(alpha_ce))


def kd_ce_loss(out_s: Tensor, out_t: Tensor, labels: Optional[Tensor], T: float, kd_weight: float = 1.0,
               ce_weight: float = 1.0, row_mask: Optional[Tensor] = None, ignore_index: int = -100,
               mse_weight: float = 0.0, mse_per_element: bool = False) -> Tensor:
    """``kd_weight * T^2 * KL(...)`` over the rows of ``row_mask`` plus
    ``ce_weight * CrossEntropy(out_s, labels)`` over the rows whose label is not
    ``ignore_index``, both means over their own row sets, in one pass over the
    logits (benchmarks/soft_target/train_kd.py:439-453;
    benchmarks/distilbert/distiller.py:719-744).  ``labels=None`` drops the CE
    term.  ``mse_weight > 0`` adds ``mse_weight * sum((out_s - out_t)^2) / rows``
    over the rows of ``row_mask`` (distiller.py:751-755; divided by the number
    of elements instead with ``mse_per_element``, as ``F.mse_loss`` does),
    accumulated into the same gradient buffer."""
    ce = float(ce_weight) if labels is not None else 0.0
    out = _host_row_loss(_KD, out_s, out_t, None, None, row_mask, labels,
                         [float(T), float(kd_weight), ce, float(mse_weight)],
                         [int(ignore_index), 1 if mse_per_element else 0])
    if out is not None:
        return out
    return _KDSoftTargetFn.apply(out_s, out_t, row_mask, float(T), float(kd_weight), labels, ce, int(ignore_index),
                                 float(mse_weight), bool(mse_per_element))


class _KDPiecesFn(torch.autograd.Function):
    """The KD (+ CE) loss on micro-batch outputs that were never concatenated:
    the kernels read every piece where it lies and write one gradient buffer
    per student piece."""

    @staticmethod
    def forward(ctx, n: int, row_mask: Optional[Tensor], labels: Optional[Tensor], T: float, weight: float,
                ce_weight: float, ignore_index: int, mse_weight: float, mse_per_element: bool, *pieces: Tensor):
        import ctypes
        s_pieces, t_pieces = pieces[:n], pieces[n:]
        _require_cuda(row_mask, labels, *pieces)
        V = int(s_pieces[0].shape[-1])
        dtype, dev = s_pieces[0].dtype, s_pieces[0].device
        s_flat, t_flat, rows = [], [], []
        for sp, tp in zip(s_pieces, t_pieces):
            if sp.shape != tp.shape or sp.dtype != dtype or tp.dtype != dtype or int(sp.shape[-1]) != V:
                raise ValueError("student/teacher pieces must agree in shape, dtype and class count")
            s2, t2 = sp.detach().reshape(-1, V), tp.detach().reshape(-1, V)
            s_flat.append(s2 if s2.is_contiguous() else s2.contiguous())
            t_flat.append(t2 if t2.is_contiguous() else t2.contiguous())
            rows.append(int(s2.shape[0]))
        total = sum(rows)
        mask_ptr = label_ptr = None
        if row_mask is not None:
            m = row_mask.detach().reshape(-1)
            if m.numel() != total:
                raise ValueError(f"row mask has {m.numel()} entries for {total} rows")
            if m.dtype != torch.bool:
                m = m != 0
            m = m.contiguous().view(torch.uint8)
            mask_ptr = m.data_ptr()
        if labels is not None:
            lab = labels.detach().reshape(-1)
            if lab.numel() != total:
                raise ValueError(f"{lab.numel()} labels for {total} rows")
            lab = (lab if lab.dtype == torch.int64 else lab.to(torch.int64)).contiguous()
            label_ptr = lab.data_ptr()
        need = [ctx.needs_input_grad[9 + i] for i in range(n)]
        grads = [torch.empty_like(s2) for s2 in s_flat] if any(need) else None
        lib = _lib.lib()
        code = _lib.dtype_code(dtype)
        ws = torch.empty(lib.ts_kd_workspace_bytes(total, V, code), dtype=torch.uint8, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])
        with _lib.on_device(dev):
            status = lib.ts_kdce_pieces_fwd_bwd(ptrs(s_flat), ptrs(t_flat), None if grads is None else ptrs(grads),
                                                (ctypes.c_int64 * n)(*rows), n, mask_ptr, label_ptr, int(ignore_index),
                                                V, 1.0 / T, T * T * weight, float(ce_weight), ws.data_ptr(),
                                                loss.data_ptr(), code, _lib.current_stream_ptr(dev))
        _lib.check(status, "ts_kdce_pieces_fwd_bwd")
        if mse_weight > 0.0:
            # the squared-error term joins loss and gradient in place, piece by piece
            ws2 = torch.empty(lib.ts_mse_workspace_bytes(total, V), dtype=torch.uint8, device=dev)
            with _lib.on_device(dev):
                status = lib.ts_mse_pieces_fwd_bwd(ptrs(s_flat), ptrs(t_flat), None if grads is None else ptrs(grads),
                                                   (ctypes.c_int64 * n)(*rows), n, mask_ptr, V, float(mse_weight),
                                                   1 if mse_per_element else 0, 1, ws2.data_ptr(), loss.data_ptr(),
                                                   code, _lib.current_stream_ptr(dev))
            _lib.check(status, "ts_mse_pieces_fwd_bwd")
        ctx.grads, ctx.need, ctx.n = grads, need, n
        ctx.shapes = [sp.shape for sp in s_pieces]
        ctx.dims = [(r, V) for r in rows]
        ctx.backward_done = False
        return loss

    @staticmethod
    def backward(ctx, grad_output: Tensor):
        none9 = (None,) * 9
        if ctx.grads is None:
            return none9 + (None,) * (2 * ctx.n)
        _once(ctx)
        outs = []
        for g, need, shape, dims in zip(ctx.grads, ctx.need, ctx.shapes, ctx.dims):
            outs.append(_scale_saved_grad(g, grad_output, *dims).view(shape) if need else None)
        return none9 + tuple(outs) + (None,) * ctx.n


def kd_ce_loss_pieces(s_pieces, t_pieces, labels: Optional[Tensor], T: float, kd_weight: float = 1.0,
                      ce_weight: float = 1.0, row_mask: Optional[Tensor] = None, ignore_index: int = -100,
                      mse_weight: float = 0.0, mse_per_element: bool = False) -> Tensor:
    """``kd_ce_loss`` on lists of micro-batch outputs (split along dim 0) that
    were never concatenated: same value as
    ``kd_ce_loss(torch.cat(s_pieces), torch.cat(t_pieces), ...)`` without either
    copy (the pipeline's gather at tspipe/gpu_task.py:147,170-171,188-191), and
    the gradient arrives per piece.  ``labels`` and ``row_mask`` cover the whole
    batch.  Up to 8 pieces per call."""
    s_pieces, t_pieces = list(s_pieces), list(t_pieces)
    if len(s_pieces) != len(t_pieces) or not s_pieces:
        raise ValueError("need as many teacher pieces as student pieces, at least one")
    n = len(s_pieces)
    return _KDPiecesFn.apply(n, row_mask, labels, float(T), float(kd_weight),
                             float(ce_weight) if labels is not None else 0.0, int(ignore_index),
                             float(mse_weight), bool(mse_per_element), *s_pieces, *t_pieces)


class _LogitsMSEFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, out_s: Tensor, out_t: Tensor, row_mask: Optional[Tensor], weight: float, per_element: bool):
        _require_cuda(out_s, out_t, row_mask)
        if out_s.shape != out_t.shape or out_s.dtype != out_t.dtype:
            raise ValueError("MSE inputs must agree in shape and dtype")
        V = int(out_s.shape[-1])
        s = out_s.detach().reshape(-1, V)
        t = out_t.detach().reshape(-1, V)
        s = s if s.is_contiguous() else s.contiguous()
        t = t if t.is_contiguous() else t.contiguous()
        rows = int(s.shape[0])
        mask_ptr = None
        if row_mask is not None:
            m = row_mask.detach().reshape(-1)
            if m.numel() != rows:
                raise ValueError(f"row mask has {m.numel()} entries for {rows} rows")
            if m.dtype != torch.bool:
                m = m != 0
            m = m.contiguous().view(torch.uint8)
            mask_ptr = m.data_ptr()
        lib = _lib.lib()
        dev = s.device
        ws = torch.empty(lib.ts_mse_workspace_bytes(rows, V), dtype=torch.uint8, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        grad = torch.empty_like(s) if ctx.needs_input_grad[0] else None
        with _lib.on_device(dev):
            status = lib.ts_mse_fwd_bwd(s.data_ptr(), t.data_ptr(), mask_ptr, rows, V, V, V, float(weight),
                                        1 if per_element else 0, 0, ws.data_ptr(), loss.data_ptr(),
                                        None if grad is None else grad.data_ptr(), V, _lib.dtype_code(s.dtype),
                                        _lib.current_stream_ptr(dev))
        _lib.check(status, "ts_mse_fwd_bwd")
        ctx.grad, ctx.shape, ctx.dims = grad, out_s.shape, (rows, V)
        ctx.backward_done = False
        return loss

    @staticmethod
    def backward(ctx, grad_output: Tensor):
        if ctx.grad is None:
            return (None,) * 5
        _once(ctx)
        return (_scale_saved_grad(ctx.grad, grad_output, *ctx.dims).view(ctx.shape),) + (None,) * 4


def logits_mse_loss(out_s: Tensor, out_t: Tensor, row_mask: Optional[Tensor] = None, weight: float = 1.0,
                    per_element: bool = True) -> Tensor:
    """Squared error between student and teacher logits.  ``per_element=True``
    is ``F.mse_loss(out_s, out_t)`` (benchmarks/soft_target/kd_losses/logits.py:17-20);
    ``per_element=False`` with a ``[bs, seq]`` mask is DistilBERT's
    ``MSELoss(reduction="sum")(s_slct, t_slct) / s_slct.size(0)``
    (benchmarks/distilbert/distiller.py:751-755)."""
    out = _host_row_loss(_MSE, out_s, out_t, None, None, row_mask, None, [float(weight)], [1 if per_element else 0])
    if out is not None:
        return out
    return _LogitsMSEFn.apply(out_s, out_t, row_mask, float(weight), bool(per_element))


class Logits(nn.Module):
    """Drop-in for benchmarks/soft_target/kd_losses/logits.py:9-20."""

    def forward(self, out_s: Tensor, out_t: Tensor) -> Tensor:
        return logits_mse_loss(out_s, out_t)


class _CosineFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: Tensor, y: Tensor, row_mask: Optional[Tensor], weight: float):
        _require_cuda(x, y, row_mask)
        if x.shape != y.shape or x.dtype != y.dtype:
            raise ValueError("cosine loss inputs must agree in shape and dtype")
        c = int(x.shape[-1])
        xs = x.detach().reshape(-1, c)
        ys = y.detach().reshape(-1, c)
        xs = xs if xs.is_contiguous() else xs.contiguous()
        ys = ys if ys.is_contiguous() else ys.contiguous()
        n = int(xs.shape[0])
        mask_ptr = None
        if row_mask is not None:
            m = row_mask.detach().reshape(-1)
            if m.numel() != n:
                raise ValueError(f"row mask has {m.numel()} entries for {n} rows")
            if m.dtype != torch.bool:
                m = m != 0
            m = m.contiguous().view(torch.uint8)
            mask_ptr = m.data_ptr()
        lib = _lib.lib()
        dev = xs.device
        ws = torch.empty(lib.ts_cosine_workspace_bytes(n), dtype=torch.uint8, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        gx = torch.empty_like(xs) if ctx.needs_input_grad[0] else None
        with _lib.on_device(dev):
            status = lib.ts_cosine_fwd_bwd(xs.data_ptr(), ys.data_ptr(), mask_ptr, n, c, weight, ws.data_ptr(),
                                           loss.data_ptr(), None if gx is None else gx.data_ptr(),
                                           _lib.dtype_code(xs.dtype), _lib.current_stream_ptr(dev))
        _lib.check(status, "ts_cosine_fwd_bwd")
        ctx.gx, ctx.shape, ctx.dims = gx, x.shape, (n, c)
        ctx.backward_done = False
        return loss

    @staticmethod
    def backward(ctx, grad_output: Tensor):
        if ctx.gx is None:
            return None, None, None, None
        _once(ctx)
        return _scale_saved_grad(ctx.gx, grad_output, *ctx.dims).view(ctx.shape), None, None, None


def cosine_embedding_loss(x: Tensor, y: Tensor, row_mask: Optional[Tensor] = None, weight: float = 1.0) -> Tensor:
    """``weight * CosineEmbeddingLoss(reduction="mean")(x[rows], y[rows], +1)`` over
    the rows (last dimension = features) kept by ``row_mask``; gradient to ``x``
    only (benchmarks/distilbert/distiller.py:756-770)."""
    out = _host_row_loss(_COSINE, x, y, None, None, row_mask, None, [float(weight)], [])
    if out is not None:
        return out
    return _CosineFn.apply(x, y, row_mask, float(weight))


class _CosinePiecesFn(torch.autograd.Function):
    """The cosine embedding loss on hidden states that were never concatenated."""

    @staticmethod
    def forward(ctx, n: int, row_mask: Optional[Tensor], weight: float, *pieces: Tensor):
        import ctypes
        x_pieces, y_pieces = pieces[:n], pieces[n:]
        _require_cuda(row_mask, *pieces)
        c = int(x_pieces[0].shape[-1])
        dtype, dev = x_pieces[0].dtype, x_pieces[0].device
        x_flat, y_flat, rows = [], [], []
        for xp, yp in zip(x_pieces, y_pieces):
            if xp.shape != yp.shape or xp.dtype != dtype or yp.dtype != dtype or int(xp.shape[-1]) != c:
                raise ValueError("the pieces of both operands must agree in shape, dtype and width")
            x2, y2 = xp.detach().reshape(-1, c), yp.detach().reshape(-1, c)
            x_flat.append(x2 if x2.is_contiguous() else x2.contiguous())
            y_flat.append(y2 if y2.is_contiguous() else y2.contiguous())
            rows.append(int(x2.shape[0]))
        total = sum(rows)
        mask_ptr = None
        if row_mask is not None:
            m = row_mask.detach().reshape(-1)
            if m.numel() != total:
                raise ValueError(f"row mask has {m.numel()} entries for {total} rows")
            if m.dtype != torch.bool:
                m = m != 0
            m = m.contiguous().view(torch.uint8)
            mask_ptr = m.data_ptr()
        need = [ctx.needs_input_grad[3 + i] for i in range(n)]
        grads = [torch.empty_like(x2) for x2 in x_flat] if any(need) else None
        lib = _lib.lib()
        ws = torch.empty(lib.ts_cosine_workspace_bytes(total), dtype=torch.uint8, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])  # noqa: E731
        with _lib.on_device(dev):
            status = lib.ts_cosine_pieces_fwd_bwd(ptrs(x_flat), ptrs(y_flat), None if grads is None else ptrs(grads),
                                                  (ctypes.c_int64 * n)(*rows), n, mask_ptr, c, float(weight),
                                                  ws.data_ptr(), loss.data_ptr(), _lib.dtype_code(dtype),
                                                  _lib.current_stream_ptr(dev))
        _lib.check(status, "ts_cosine_pieces_fwd_bwd")
        ctx.grads, ctx.need, ctx.n = grads, need, n
        ctx.shapes = [xp.shape for xp in x_pieces]
        ctx.dims = [(r, c) for r in rows]
        ctx.backward_done = False
        return loss

    @staticmethod
    def backward(ctx, grad_output: Tensor):
        if ctx.grads is None:
            return (None,) * (3 + 2 * ctx.n)
        _once(ctx)
        outs = []
        for g, need, shape, dims in zip(ctx.grads, ctx.need, ctx.shapes, ctx.dims):
            outs.append(_scale_saved_grad(g, grad_output, *dims).view(shape) if need else None)
        return (None,) * 3 + tuple(outs) + (None,) * ctx.n


def cosine_embedding_loss_pieces(x_pieces, y_pieces, row_mask: Optional[Tensor] = None, weight: float = 1.0) -> Tensor:
    """``cosine_embedding_loss`` on lists of micro-batch outputs (split along
    dim 0) that were never concatenated; ``row_mask`` covers the whole batch.
    Up to 8 pieces per call."""
    x_pieces, y_pieces = list(x_pieces), list(y_pieces)
    if len(x_pieces) != len(y_pieces) or not x_pieces:
        raise ValueError("need as many teacher pieces as student pieces, at least one")
    return _CosinePiecesFn.apply(len(x_pieces), row_mask, float(weight), *x_pieces, *y_pieces)


# ---------------------------------------------------------------------------
# BYOL normalised MSE
# ---------------------------------------------------------------------------

class _BYOLFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1: Tensor, y1: Tensor, x2: Optional[Tensor], y2: Optional[Tensor]):
        _require_cuda(x1, y1, x2, y2)
        tensors = [x1, y1] + ([x2, y2] if x2 is not None else [])
        if any(t.dim() != 2 for t in tensors):
            raise ValueError("BYOL loss expects [batch, features] projections")
        if any(t.shape != x1.shape or t.dtype != x1.dtype for t in tensors):
            raise ValueError("BYOL loss inputs must agree in shape and dtype")
        n, c = int(x1.shape[0]), int(x1.shape[1])
        prep = [t.detach() if t.is_contiguous() else t.detach().contiguous() for t in tensors]
        dev = x1.device
        ws = torch.empty(2 * max(n, 1), dtype=torch.float32, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        g1 = torch.empty_like(prep[0]) if ctx.needs_input_grad[0] else None
        g2 = torch.empty_like(prep[2]) if (x2 is not None and ctx.needs_input_grad[2]) else None
        with _lib.on_device(dev):
            status = _lib.lib().ts_byol_fwd_bwd(
                prep[0].data_ptr(), prep[1].data_ptr(),
                prep[2].data_ptr() if x2 is not None else None,
                prep[3].data_ptr() if x2 is not None else None, n, c, ws.data_ptr(), loss.data_ptr(),
                None if g1 is None else g1.data_ptr(), None if g2 is None else g2.data_ptr(),
                _lib.dtype_code(x1.dtype), _lib.current_stream_ptr(dev))
        _lib.check(status, "ts_byol_fwd_bwd")
        ctx.g1, ctx.g2, ctx.dims = g1, g2, (n, c)
        ctx.backward_done = False
        return loss

    @staticmethod
    def backward(ctx, grad_output: Tensor):
        _once(ctx)
        # the context lets go of the buffers, so autograd can adopt them as .grad instead of copying
        g1, g2 = ctx.g1, ctx.g2
        ctx.g1 = ctx.g2 = None
        out1 = out2 = None
        if g1 is not None:
            out1 = _scale_saved_grad(g1, grad_output, *ctx.dims)
        if g2 is not None:
            out2 = _scale_saved_grad(g2, grad_output, *ctx.dims)
        return out1, None, out2, None


def byol_loss(online_view_1: Tensor, online_view_2: Tensor, target_view_1: Tensor,
              target_view_2: Tensor) -> Tensor:
    """``mean(rl(o1, t2) + rl(o2, t1))`` with ``rl(x, y) = 2 - 2 <x^, y^>``
    (benchmarks/byol/trainer.py:51-55, 192-196)."""
    out = _host_row_loss(_BYOL, online_view_1, target_view_2, online_view_2, target_view_1, None, None, [], [])
    if out is not None:
        return out
    return _BYOLFn.apply(online_view_1, target_view_2, online_view_2, target_view_1)


def regression_loss_mean(x: Tensor, y: Tensor) -> Tensor:
    """``regression_loss(x, y).mean()`` for a single pair (benchmarks/byol/trainer.py:51-55)."""
    out = _host_row_loss(_BYOL, x, y, None, None, None, None, [], [])
    if out is not None:
        return out
    return _BYOLFn.apply(x, y, None, None)


# ---------------------------------------------------------------------------
# MoCo-v3 InfoNCE
# ---------------------------------------------------------------------------

class _InfoNCEFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q1: Tensor, k1: Tensor, q2: Optional[Tensor], k2: Optional[Tensor], tau: float):
        _require_cuda(q1, k1, q2, k2)
        tensors = [q1, k1] + ([q2, k2] if q2 is not None else [])
        if any(t.dim() != 2 for t in tensors):
            raise ValueError("InfoNCE expects [batch, features] embeddings")
        if any(t.shape != q1.shape or t.dtype != q1.dtype for t in tensors):
            raise ValueError("InfoNCE inputs must agree in shape and dtype")
        n, c_in = int(q1.shape[0]), int(q1.shape[1])
        if c_in > 512:
            raise ValueError(f"InfoNCE kernels take embeddings of up to 512 features, got {c_in}")
        if not tau > 0:
            raise ValueError(f"InfoNCE needs a positive temperature, got {tau}")
        prep = [t.detach() if t.is_contiguous() else t.detach().contiguous() for t in tensors]
        # bf16 / fp16 embeddings at temperatures of 0.03 and above run on the bf16 matrix cores, whose
        # kernels come in widths 64, 128 and 256: narrower rows are padded (zero features change neither
        # norms nor products).  fp32 embeddings, wider rows and smaller temperatures take the fp32
        # kernels, which accept any width as it is.
        c = c_in
        if q1.dtype != torch.float32 and tau >= 0.03 and c_in <= 256:
            c = 64 if c_in <= 64 else 128 if c_in <= 128 else 256
            if c != c_in:
                prep = [torch.nn.functional.pad(t, (0, c - c_in)) for t in prep]
        dev = q1.device
        lib = _lib.lib()
        pairs = 2 if q2 is not None else 1
        ws = torch.empty(lib.ts_infonce_workspace_bytes(n, c, pairs), dtype=torch.uint8, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        g1 = torch.empty_like(prep[0]) if ctx.needs_input_grad[0] else None
        g2 = torch.empty_like(prep[2]) if (q2 is not None and ctx.needs_input_grad[2]) else None
        with _lib.on_device(dev):
            status = lib.ts_infonce_fwd_bwd(
                prep[0].data_ptr(), prep[1].data_ptr(),
                prep[2].data_ptr() if q2 is not None else None,
                prep[3].data_ptr() if q2 is not None else None, n, c, tau, ws.data_ptr(), loss.data_ptr(),
                None if g1 is None else g1.data_ptr(), None if g2 is None else g2.data_ptr(),
                _lib.dtype_code(q1.dtype), _lib.current_stream_ptr(dev))
        _lib.check(status, "ts_infonce_fwd_bwd")
        ctx.g1, ctx.g2, ctx.dims, ctx.c_in = g1, g2, (n, c), c_in
        ctx.backward_done = False
        return loss

    @staticmethod
    def backward(ctx, grad_output: Tensor):
        _once(ctx)
        # the context lets go of the buffers, so autograd can adopt them as .grad instead of copying
        g1, g2 = ctx.g1, ctx.g2
        ctx.g1 = ctx.g2 = None
        out1 = out2 = None
        if g1 is not None:
            out1 = _scale_saved_grad(g1, grad_output, *ctx.dims)
            out1 = out1 if ctx.c_in == ctx.dims[1] else out1[:, :ctx.c_in]
        if g2 is not None:
            out2 = _scale_saved_grad(g2, grad_output, *ctx.dims)
            out2 = out2 if ctx.c_in == ctx.dims[1] else out2[:, :ctx.c_in]
        return out1, None, out2, None, None


def _infonce(q1: Tensor, k1: Tensor, q2: Optional[Tensor], k2: Optional[Tensor], tau: float) -> Tensor:
    """The plain case (dense 2-D device tensors, 64 / 128 / 256 features) goes
    to the C++ autograd node of the host helper, whose backward needs no
    interpreter lock; everything else, and every error, to the Python one."""
    host = _lib.host_helper()
    if host is not None and type(q1) is Tensor and q1.is_cuda and hasattr(host, "infonce"):
        out = host.infonce(q1, k1, q2, k2, tau, _lib.current_stream_ptr(q1.device))
        if out is not None:
            return out
    return _InfoNCEFn.apply(q1, k1, q2, k2, tau)


def set_infonce_workgroup_target(workgroups: int = 0) -> int:
    """Scheduling knob of the InfoNCE kernels (``ts_infonce_set_workgroup_target``):
    about how many workgroups the main kernel puts on the 256 CUs.  The default
    (0 or 256) suits a loss that has the GPU to itself; a pipeline that runs the
    loss beside bandwidth-bound work on another stream, as TSPipe runs it beside
    the momentum update (tspipe/gpu_task.py:385-410), gets a shorter step from
    32 to 64: fewer partial sums through HBM, CUs left to the other stream.
    Process-wide; returns the previous value."""
    return int(_lib.lib().ts_infonce_set_workgroup_target(int(workgroups)))


def set_infonce_fp32_arithmetic(on: bool = True) -> bool:
    """Accuracy switch of the InfoNCE kernels (``ts_infonce_set_fp32_arithmetic``):
    when on, bf16 / fp16 embeddings also run on the fp32-MFMA kernels (every
    product and sum in fp32, as the reference's fp32 run,
    benchmarks/moco-v3/main.py:149-160), about seven times slower than the
    bf16-MFMA kernels.  Meant for nearly aligned (q, k) pairs, where the bf16
    kernels' rounding of the negatives' weights shows in the gradient.
    Process-wide; returns the previous setting."""
    return bool(_lib.lib().ts_infonce_set_fp32_arithmetic(1 if on else 0))


def infonce_loss(q: Tensor, k: Tensor, tau: float) -> Tensor:
    """One direction of MoCo-v3's loss: ``CE(q^ k^T / tau, arange(N)) * 2 tau``
    (benchmarks/moco-v3/main.py:149-160)."""
    return _infonce(q, k, None, None, float(tau))


def moco_contrastive_loss_pair(online_view_1: Tensor, online_view_2: Tensor, target_view_1: Tensor,
                               target_view_2: Tensor, tau: float) -> Tensor:
    """``loss(o1, t2) + loss(o2, t1)`` in one launch (benchmarks/moco-v3/main.py:162)."""
    return _infonce(online_view_1, target_view_2, online_view_2, target_view_1, float(tau))


# ---------------------------------------------------------------------------
# The self-supervised losses on micro-batch outputs that were never gathered
# ---------------------------------------------------------------------------

class _PairPiecesFn(torch.autograd.Function):
    """InfoNCE or BYOL loss over two (student, teacher) pairs whose operands
    come as lists of micro-batch pieces (split along dim 0): the kernels read
    every piece where it lies and write one gradient buffer per student piece,
    so neither ``torch.cat`` of tspipe/gpu_task.py:188-191 is needed."""

    @staticmethod
    def forward(ctx, kind: str, n: int, tau: float, *pieces: Tensor):
        import ctypes
        o1, t2, o2, t1 = (pieces[i * n:(i + 1) * n] for i in range(4))  # pairs (o1, t2) and (o2, t1)
        _require_cuda(*pieces)
        first = o1[0]
        c, dtype, dev = int(first.shape[1]), first.dtype, first.device
        rows = []
        for group in zip(o1, t2, o2, t1):
            if any(t.dim() != 2 or t.shape != group[0].shape or t.dtype != dtype for t in group) or \
                    int(group[0].shape[1]) != c:
                raise ValueError("the pieces of all four operands must agree in shape and dtype, piece by piece")
            rows.append(int(group[0].shape[0]))
        total = sum(rows)
        dense = [[t.detach() if t.is_contiguous() else t.detach().contiguous() for t in grp] for grp in (o1, t2, o2, t1)]
        need1 = [ctx.needs_input_grad[3 + i] for i in range(n)]
        need2 = [ctx.needs_input_grad[3 + 2 * n + i] for i in range(n)]
        g1 = [torch.empty_like(t) for t in dense[0]] if any(need1) else None
        g2 = [torch.empty_like(t) for t in dense[2]] if any(need2) else None
        lib = _lib.lib()
        code = _lib.dtype_code(dtype)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        ptrs = lambda ts: None if ts is None else (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])  # noqa: E731
        rows_arr = (ctypes.c_int64 * n)(*rows)
        with _lib.on_device(dev):
            stream = _lib.current_stream_ptr(dev)
            if kind == "infonce":
                if c > 512:
                    raise ValueError(f"InfoNCE kernels take embeddings of up to 512 features, got {c}")
                if not tau > 0:
                    raise ValueError(f"InfoNCE needs a positive temperature, got {tau}")
                ws = torch.empty(lib.ts_infonce_workspace_bytes(total, c, 2), dtype=torch.uint8, device=dev)
                status = lib.ts_infonce_pieces_fwd_bwd(ptrs(dense[0]), ptrs(dense[1]), ptrs(g1), ptrs(dense[2]),
                                                       ptrs(dense[3]), ptrs(g2), rows_arr, n, c, tau, ws.data_ptr(),
                                                       loss.data_ptr(), code, stream)
                _lib.check(status, "ts_infonce_pieces_fwd_bwd")
            else:
                ws = torch.empty(2 * max(total, 1), dtype=torch.float32, device=dev)
                status = lib.ts_byol_pieces_fwd_bwd(ptrs(dense[0]), ptrs(dense[1]), ptrs(g1), ptrs(dense[2]),
                                                    ptrs(dense[3]), ptrs(g2), rows_arr, n, c, ws.data_ptr(),
                                                    loss.data_ptr(), code, stream)
                _lib.check(status, "ts_byol_pieces_fwd_bwd")
        ctx.g1, ctx.g2, ctx.need1, ctx.need2, ctx.n = g1, g2, need1, need2, n
        ctx.dims = [(r, c) for r in rows]
        ctx.backward_done = False
        return loss

    @staticmethod
    def backward(ctx, grad_output: Tensor):
        _once(ctx)
        n = ctx.n
        g1, g2 = ctx.g1, ctx.g2
        ctx.g1 = ctx.g2 = None
        out1 = [None] * n if g1 is None else [
            _scale_saved_grad(g, grad_output, *d) if need else None for g, need, d in zip(g1, ctx.need1, ctx.dims)]
        out2 = [None] * n if g2 is None else [
            _scale_saved_grad(g, grad_output, *d) if need else None for g, need, d in zip(g2, ctx.need2, ctx.dims)]
        return (None, None, None) + tuple(out1) + (None,) * n + tuple(out2) + (None,) * n


def _pair_pieces(kind: str, o1, o2, t1, t2, tau: float) -> Tensor:
    o1, o2, t1, t2 = list(o1), list(o2), list(t1), list(t2)
    n = len(o1)
    if n == 0 or any(len(x) != n for x in (o2, t1, t2)):
        raise ValueError("need the same number of pieces, at least one, for all four operands")
    return _PairPiecesFn.apply(kind, n, float(tau), *o1, *t2, *o2, *t1)


def moco_contrastive_loss_pieces(online_view_1, online_view_2, target_view_1, target_view_2, args,
                                 extra_args) -> Tensor:
    """``moco_contrastive_loss`` for a pipeline that hands over the lists of
    micro-batch outputs instead of gathering them first (the ``torch.cat`` at
    tspipe/gpu_task.py:188-191): each argument is a list of ``[rows_i, C]``
    pieces, the same split for all four.  Same value as the loss on the
    concatenated tensors; the gradient arrives per student piece."""
    return _pair_pieces("infonce", online_view_1, online_view_2, target_view_1, target_view_2,
                        float(extra_args.moco_t))


def byol_contrastive_loss_pieces(online_view_1, online_view_2, target_view_1, target_view_2,
                                 args: Namespace = None, extra_args: Namespace = None) -> Tensor:
    """``byol_contrastive_loss`` on lists of micro-batch pieces, as above."""
    return _pair_pieces("byol", online_view_1, online_view_2, target_view_1, target_view_2, 0.0)


# ---------------------------------------------------------------------------
# loss_fn plug-ins with the reference's signatures
# ---------------------------------------------------------------------------

def byol_contrastive_loss(online_view_1, online_view_2, target_view_1, target_view_2,
                          args: Namespace = None, extra_args: Namespace = None) -> Tensor:
    """``TSPipeBYOLTrainer.contrastive_loss`` (benchmarks/byol/trainer.py:192-196)."""
    return byol_loss(online_view_1, online_view_2, target_view_1, target_view_2)


def moco_contrastive_loss(online_view_1, online_view_2, target_view_1, target_view_2, args, extra_args) -> Tensor:
    """``contrastive_loss`` of benchmarks/moco-v3/main.py:147-162; the
    temperature comes from ``extra_args.moco_t``."""
    return moco_contrastive_loss_pair(online_view_1, online_view_2, target_view_1, target_view_2,
                                      float(extra_args.moco_t))


def soft_target_tspipe_loss(model_out: Tensor, ema_model_out: Tensor, label: Tensor, tspipe_args, args,
                            epoch: int) -> Tensor:
    """``tspipe_loss`` of benchmarks/soft_target/train_kd.py:439-453: hard-label
    cross entropy plus ``lambda_kd`` times the KD criterion -- the soft-target
    KL for ``args.kd_mode == 'st'`` (both in one kernel pass), the logits MSE
    for ``'logits'``."""
    mode = getattr(args, "kd_mode", "st")
    if mode == "st":
        return kd_ce_loss(model_out, ema_model_out.detach(), label, args.T, kd_weight=args.lambda_kd, ce_weight=1.0)
    if mode == "logits":
        return kd_ce_loss(model_out, ema_model_out.detach(), label, 1.0, kd_weight=0.0, ce_weight=1.0,
                          mse_weight=args.lambda_kd, mse_per_element=True)
    raise AssertionError(f"kd_mode {mode!r}: the reference knows 'st' and 'logits'")


def _ce_terms(lm_labels: Tensor, params):
    """The hard-label terms of DistilBERT's loss as (labels, weight) pairs:
    masked-LM cross entropy against ``lm_labels`` (distiller.py:742-744) and
    causal-LM cross entropy, where the logits at position p are scored against
    the label at p+1 and the last position of a sequence has no target
    (distiller.py:745-749)."""
    terms = []
    alpha_mlm = float(getattr(params, "alpha_mlm", 0.0))
    alpha_clm = float(getattr(params, "alpha_clm", 0.0))
    if alpha_mlm > 0.0:
        terms.append((lm_labels, alpha_mlm))
    if alpha_clm > 0.0:
        shifted = torch.full_like(lm_labels, -100)
        shifted[..., :-1] = lm_labels[..., 1:]
        terms.append((shifted, alpha_clm))
    return terms


def distil_loss_fn(student_outputs, teacher_outputs, labels, tspipe_args, params, epoch: int) -> Tensor:
    """``TSPipeDistiller.loss_fn`` of benchmarks/distilbert/distiller.py:711-772:
    ``alpha_ce`` x masked KD, ``alpha_mlm`` x masked-LM cross entropy and/or
    ``alpha_clm`` x causal-LM cross entropy (ignore_index -100) -- the first of
    the two in the same pass over the logits as the KD term, a second one in a
    pass of its own -- ``alpha_mse`` x squared error of the selected
    logits, and ``alpha_cos`` x cosine embedding loss on the last hidden states.  ``params`` carries
    ``alpha_ce, alpha_mlm, alpha_clm, alpha_mse, alpha_cos, temperature,
    restrict_ce_to_mask`` like the reference's LossComputeParam."""
    s_logits, t_logits = student_outputs["logits"], teacher_outputs["logits"]
    lm_labels, attention_mask = labels
    alpha_mse = float(getattr(params, "alpha_mse", 0.0))
    mask = (lm_labels > -1) if params.restrict_ce_to_mask else attention_mask
    terms = _ce_terms(lm_labels, params)
    ce_labels, ce_weight = terms[0] if terms else (None, 0.0)
    loss = kd_ce_loss(s_logits, t_logits, ce_labels, params.temperature, kd_weight=params.alpha_ce,
                      ce_weight=ce_weight, row_mask=mask, ignore_index=-100, mse_weight=alpha_mse)
    for ce_labels, ce_weight in terms[1:]:
        # both alpha_mlm and alpha_clm set (distiller.py:742-749 adds both terms): the
        # second cross entropy is a pass of its own over the student logits
        loss = loss + kd_ce_loss(s_logits, t_logits, ce_labels, params.temperature, kd_weight=0.0,
                                 ce_weight=ce_weight, row_mask=mask, ignore_index=-100)
    if getattr(params, "alpha_cos", 0.0) > 0.0:
        s_hid = student_outputs["hidden_states"][-1]
        t_hid = teacher_outputs["hidden_states"][-1]
        loss = loss + cosine_embedding_loss(s_hid, t_hid, attention_mask, params.alpha_cos)
    return loss


def distil_loss_fn_pieces(student_pieces, teacher_pieces, labels, tspipe_args, params, epoch: int) -> Tensor:
    """``distil_loss_fn`` for a pipeline that hands over the per-micro-batch
    output dicts instead of gathering them first (tspipe/gpu_task.py:147,
    170-171, 188-191 is where the reference concatenates).  Every term reads
    the pieces where they lie: the logits through ``kd_ce_loss_pieces`` (KD,
    cross entropy and the ``alpha_mse`` squared error), the last hidden states
    through ``cosine_embedding_loss_pieces``.  ``labels`` is the whole batch's
    ``(lm_labels, attention_mask)`` as in ``distil_loss_fn``."""
    lm_labels, attention_mask = labels
    alpha_mse = float(getattr(params, "alpha_mse", 0.0))
    mask = (lm_labels > -1) if params.restrict_ce_to_mask else attention_mask
    terms = _ce_terms(lm_labels, params)
    ce_labels, ce_weight = terms[0] if terms else (None, 0.0)
    s_list, t_list = [p["logits"] for p in student_pieces], [p["logits"] for p in teacher_pieces]
    loss = kd_ce_loss_pieces(s_list, t_list, ce_labels, params.temperature, kd_weight=params.alpha_ce,
                             ce_weight=ce_weight, row_mask=mask, ignore_index=-100, mse_weight=alpha_mse)
    for ce_labels, ce_weight in terms[1:]:
        loss = loss + kd_ce_loss_pieces(s_list, t_list, ce_labels, params.temperature, kd_weight=0.0,
                                        ce_weight=ce_weight, row_mask=mask, ignore_index=-100)
    if getattr(params, "alpha_cos", 0.0) > 0.0:
        loss = loss + cosine_embedding_loss_pieces([p["hidden_states"][-1] for p in student_pieces],
                                                   [p["hidden_states"][-1] for p in teacher_pieces],
                                                   attention_mask, params.alpha_cos)
    return loss

