"""Micro-batch scatter / gather with the interface of tspipe/batch_ops.py.

``scatter`` keeps the reference's zero-copy behaviour (``Tensor.chunk`` views,
batch_ops.py:168-183); ``gather`` (``torch.cat`` on dim 0, batch_ops.py:186-205)
runs as one launch of the multi-segment copy kernel however many pieces and
positions there are.  ``scatter_copy`` is the owning form of scatter for
callers that need contiguous, independently freeable micro-batches.

``Batch`` (batch_ops.py:24-150), ``check`` (152-165), ``ScatterGatherFn`` /
``batch_size`` / ``defaultScatterGatherFn`` (208-221) keep their names,
arguments and exceptions so existing plug-ins work unchanged.
"""
from dataclasses import dataclass
from typing import Any, Callable, Iterator, List, Sequence, Tuple, Union

import torch
from torch import Tensor

from . import _lib, _tables
from .utils import traverse_tensor_map

Tensors = Union[Tuple[Tensor, ...], dict]
TensorOrTensors = Union[Tensor, Tensors]


class Batch:
    """One micro-batch: a single tensor ("atomic") or a tuple of tensors."""

    def __init__(self, value: TensorOrTensors) -> None:
        self.value = value
        self.atomic = torch.is_tensor(value)
        self.debug_info = ""

    # -- whole-batch transforms ------------------------------------------------
    def to_(self, device: torch.device) -> "Batch":
        self.value = traverse_tensor_map(self.value, lambda t: t.to(device=device))
        return self

    def clone(self) -> "Batch":
        return Batch(traverse_tensor_map(self.value, lambda t: t.clone()))

    def detach(self) -> "Batch":
        return Batch(traverse_tensor_map(self.value, lambda t: t.detach()))

    def share_memory_(self) -> "Batch":
        self.value.share_memory_()
        return self

    def pin_memory(self) -> "Batch":
        return Batch(self.value.pin_memory())

    def call(self, function: Callable[[TensorOrTensors], TensorOrTensors]) -> "Batch":
        return Batch(function(self.value))

    # -- typed accessors -------------------------------------------------------
    @property
    def tensor(self) -> Tensor:
        if not self.atomic:
            raise AttributeError("not atomic batch")
        return self.value

    @property
    def tensors(self) -> Tensors:
        if self.atomic:
            raise AttributeError("batch is atomic")
        return self.value

    @property
    def tensor_or_tensors(self) -> TensorOrTensors:
        return self.value

    # -- container protocol ----------------------------------------------------
    def __repr__(self) -> str:
        return f"Batch[atomic={self.atomic!r}]({self.value!r})"

    def __iter__(self) -> Iterator[Tensor]:
        if self.atomic:
            yield self.value
        else:
            yield from self.value

    def __len__(self) -> int:
        return 1 if self.atomic else len(self.value)

    def __getitem__(self, index: int) -> Tensor:
        if not self.atomic:
            return self.value[index]
        if index != 0:
            raise IndexError("atomic batch allows index 0 only")
        return self.value

    def __setitem__(self, index: Union[int, slice], value: TensorOrTensors) -> None:
        if isinstance(index, int):
            if self.atomic:
                if index != 0:
                    raise IndexError("atomic batch allows index 0 only")
                self.value = value
            else:
                self.value = self.value[:index] + (value,) + self.value[index + 1:]
            return
        if not (index.start is index.stop is index.step is None):
            raise NotImplementedError("only slice [:] supported")
        if not self.atomic:
            self.value = value
        elif len(value) != 1:
            raise IndexError("atomic batch cannot be replaced with multiple tensors")
        else:
            self.value = value[0]


def check(input: Any) -> None:
    """Raises ``TypeError`` unless ``input`` is a tensor or a (nested) tuple of tensors."""
    if isinstance(input, tuple):
        for item in input:
            check(item)
    elif not isinstance(input, Tensor):
        raise TypeError(f"expected Tensor, but got {input.__class__.__name__}")


# ---------------------------------------------------------------------------
# dim-0 concatenation on the device: one launch for any number of outputs
# ---------------------------------------------------------------------------

def _cat_plan(pieces: Sequence[Tensor]) -> Tuple[Tensor, List[Tensor], List[int], List[int]]:
    """Allocates the result of concatenating ``pieces``; lists the source
    tensors, their destination addresses inside the result and byte counts."""
    first = pieces[0]
    if any(not torch.is_tensor(p) for p in pieces):
        raise TypeError("gather expects tensors")
    if first.dim() == 0:
        raise RuntimeError("zero-dimensional tensor cannot be concatenated")
    if not first.is_cuda:
        raise TypeError("tspipe_amd gather runs on device tensors only (no host fallback)")
    tail = first.shape[1:]
    for p in pieces:
        if p.shape[1:] != tail or p.dtype != first.dtype or p.device != first.device:
            raise RuntimeError(
                f"gather: pieces must agree in trailing shape, dtype and device "
                f"(got {tuple(p.shape)} {p.dtype} vs {tuple(first.shape)} {first.dtype})")
    rows = [int(p.shape[0]) for p in pieces]
    out = torch.empty((sum(rows),) + tuple(tail), dtype=first.dtype, device=first.device)
    # destination addresses by arithmetic: a view of `out` per piece costs more host time than the
    # copy of a small piece takes
    row_bytes = (out.numel() // out.shape[0] if out.shape[0] else 0) * out.element_size()
    base = out.data_ptr()
    srcs, dsts, sizes, r0 = [], [], [], 0
    for p, r in zip(pieces, rows):
        if r:
            srcs.append(p if p.is_contiguous() else p.detach().contiguous())
            dsts.append(base + r0 * row_bytes)
            sizes.append(r * row_bytes)
        r0 += r
    return out, srcs, dsts, sizes


class _CatMany(torch.autograd.Function):
    """cat(dim 0) of several groups in one launch; backward hands out views of
    the incoming gradients (zero-copy), which is what torch.cat's backward
    (narrow) does."""

    @staticmethod
    def forward(ctx, group_sizes: Tuple[int, ...], *pieces: Tensor):
        outs, srcs, dsts, sizes, rows = [], [], [], [], []
        i = 0
        for g in group_sizes:
            group = pieces[i:i + g]
            i += g
            out, s, d, b = _cat_plan(group)
            outs.append(out)
            srcs += s
            dsts += d
            sizes += b
            rows.append([int(p.shape[0]) for p in group])
        dev = outs[0].device
        src_ptrs = [t.data_ptr() for t in srcs]  # `srcs` keeps contiguous copies alive until the launch is enqueued
        if dev.index == torch.cuda.current_device():
            _tables.copy_segments_raw(src_ptrs, dsts, sizes, dev)
        else:
            with _lib.on_device(dev):
                _tables.copy_segments_raw(src_ptrs, dsts, sizes, dev)
        ctx.rows = rows
        return tuple(outs)

    @staticmethod
    def backward(ctx, *grads: Tensor):
        result: List[Any] = [None]
        for g, rows in zip(grads, ctx.rows):
            r0 = 0
            for r in rows:
                result.append(None if g is None else g[r0:r0 + r])
                r0 += r
        return tuple(result)


def concat_groups(groups: Sequence[Sequence[Tensor]]) -> List[Tensor]:
    """``[torch.cat(g) for g in groups]`` as a single kernel launch."""
    groups = [tuple(g) for g in groups]
    if not groups:
        return []
    flat = [p for g in groups for p in g]
    return list(_CatMany.apply(tuple(len(g) for g in groups), *flat))


def concat_dim0(pieces: Sequence[Tensor]) -> Tensor:
    """``torch.cat(pieces)`` through the copy kernel."""
    return concat_groups([pieces])[0]


def scatter(input: TensorOrTensors, chunks: int) -> List[Batch]:
    """Splits a mini-batch into micro-batches (views; batch_ops.py:168-183).

    ``Tensor.chunk`` rules apply: pieces have ``ceil(N/chunks)`` rows, fewer
    than ``chunks`` pieces may come back, and tuples are zipped position-wise
    (truncating to the shortest member)."""
    if isinstance(input, Tensor):
        return [Batch(piece) for piece in input.chunk(chunks)]
    per_position = [member.chunk(chunks) for member in input]
    return [Batch(group) for group in zip(*per_position)]


def scatter_copy(input: TensorOrTensors, chunks: int) -> List[Batch]:
    """Owning form of :func:`scatter`: every micro-batch gets its own
    contiguous storage, all filled by one multi-segment copy launch."""
    views = scatter(input, chunks)
    srcs = [t for b in views for t in b]
    if not srcs:
        return views
    if any(not t.is_cuda for t in srcs):
        raise TypeError("tspipe_amd scatter_copy runs on device tensors only (no host fallback)")
    dsts = [torch.empty_like(t, memory_format=torch.contiguous_format) for t in srcs]
    live = [(s.detach() if s.is_contiguous() else s.detach().contiguous(), d)
            for s, d in zip(srcs, dsts) if s.numel()]
    with _lib.on_device(srcs[0].device):
        _tables.copy_segments([s for s, _ in live], [d for _, d in live])
    it = iter(dsts)
    return [Batch(next(it)) if b.atomic else Batch(tuple(next(it) for _ in b)) for b in views]


def gather(outputs: List[Batch]) -> TensorOrTensors:
    """Concatenates micro-batches into a mini-batch (batch_ops.py:186-205)."""
    if outputs[0].atomic:
        return concat_dim0(tuple(b.tensor for b in outputs))
    per_position = zip(*(b.tensors for b in outputs))
    return tuple(concat_groups(list(per_position)))


@dataclass
class ScatterGatherFn:
    scatter: Callable[[TensorOrTensors, int], List[Batch]]
    gather: Callable[[List[Batch]], TensorOrTensors]
    batch_size: Callable[[TensorOrTensors], int]


def batch_size(t: TensorOrTensors) -> int:
    if torch.is_tensor(t):
        return t.shape[0]
    raise NotImplementedError()


defaultScatterGatherFn = ScatterGatherFn(scatter=scatter, gather=gather, batch_size=batch_size)


# Structure-aware variant, as the DistilBERT benchmark defines it
# (benchmarks/distilbert/distiller.py:774-836).

def generic_scatter(input: Any, chunks: int) -> List[Batch]:
    from .utils import generic_object_scatter
    return [Batch(piece) for piece in generic_object_scatter(input, chunks)]


def generic_gather(outputs: List[Batch]) -> Any:
    from .utils import generic_object_gather
    if outputs[0].atomic:
        return concat_dim0(tuple(b.tensor for b in outputs))
    return generic_object_gather(*(b.value for b in outputs))
