"""Structure-aware micro-batch split / merge for nested model inputs and outputs.

Host-side mirror of tspipe/utils.py:179-200 (``traverse_tensor_map``) and
tspipe/utils.py:225-292 (``generic_object_scatter`` / ``generic_object_gather``),
which the DistilBERT benchmark plugs into its ``ScatterGatherFn``
(benchmarks/distilbert/distiller.py:774-836).  Tensor leaves are split into
dim-0 views and merged by the multi-segment copy kernel; everything else is
structure bookkeeping whose quirks are kept:

* ``dict`` is tested before ``OrderedDict`` when scattering, so an
  ``OrderedDict`` comes back as plain ``dict`` pieces (utils.py:231 vs 236);
* containers are recombined with ``zip``, so the number of pieces is that of
  the leaf yielding the fewest (``Tensor.chunk`` may return fewer than asked);
* non-tensor leaves are replicated on scatter and must compare equal on gather.
"""
from collections import OrderedDict
from typing import Any, Callable

from torch import Tensor

from ._outputs import TSPipeModelOutput


def traverse_tensor_map(obj: Any, fn: Callable[[Tensor], Any]) -> Any:
    """Rebuilds ``obj`` with ``fn`` applied to every tensor leaf (utils.py:179-200)."""

    def walk(o):
        if isinstance(o, list):
            return [walk(c) for c in o]
        if isinstance(o, OrderedDict):
            return OrderedDict((k, walk(v)) for k, v in o.items())
        if isinstance(o, dict):
            return {k: walk(v) for k, v in o.items()}
        if isinstance(o, (tuple, zip)):
            return tuple(walk(c) for c in o)
        if isinstance(o, Tensor):
            return fn(o)
        return o

    if isinstance(obj, TSPipeModelOutput):
        return obj.with_data(walk(obj.data))
    return walk(obj)


def generic_object_scatter(obj: Any, chunks: int) -> Any:
    """Splits every tensor leaf into ``chunks`` dim-0 views and returns the
    per-piece structures (utils.py:225-254)."""

    def split(o):
        if isinstance(o, list):
            return [list(piece) for piece in zip(*(split(c) for c in o))]
        if isinstance(o, tuple):
            return tuple(zip(*(split(c) for c in o)))
        if isinstance(o, dict):  # also catches OrderedDict: pieces are plain dicts
            key_pieces = zip(*(split(k) for k in o.keys()))
            val_pieces = zip(*(split(v) for v in o.values()))
            return tuple(dict(zip(ks, vs)) for ks, vs in zip(key_pieces, val_pieces))
        if isinstance(o, Tensor):
            return o.chunk(chunks)
        return [o for _ in range(chunks)]

    if isinstance(obj, TSPipeModelOutput):
        return [obj.with_data(piece) for piece in split(obj.data)]
    return split(obj)


class _Pending:
    """Stand-in for a tensor leaf whose concatenation is still to be launched."""
    __slots__ = ("index",)

    def __init__(self, index: int):
        self.index = index


def generic_object_gather(*objs: Any) -> Any:
    """Merges structures produced by ``generic_object_scatter`` (utils.py:256-292).

    The structure is walked first (all type, key and value checks happen
    there, in the reference's order), the tensor leaves are only collected;
    then every leaf of the whole structure is concatenated by ONE copy launch
    and the results are put in place."""
    from . import batch_ops

    groups = []

    def keys_agree(first, others):
        for other in others:
            if any(a != b for a, b in zip(first.keys(), other.keys())):
                raise ValueError(f"Key of given objects must match: {first} != {other}")

    def merge(*items):
        if not items:
            return tuple()
        head = items[0]
        if any(type(head) != type(x) for x in items):
            raise ValueError(f"Type of given objects must match: {[type(x) for x in items]}")
        if isinstance(head, list):
            return [merge(*group) for group in zip(*items)]
        if isinstance(head, (tuple, zip)):
            return tuple(merge(*group) for group in zip(*items))
        if isinstance(head, dict):
            keys_agree(head, items)
            merged = ((group[0][0], merge(*(kv[1] for kv in group)))
                      for group in zip(*(x.items() for x in items)))
            return OrderedDict(merged) if isinstance(head, OrderedDict) else dict(merged)
        if isinstance(head, Tensor):
            groups.append(items)
            return _Pending(len(groups) - 1)
        if any(head != x for x in items):
            raise ValueError(f"Value of given objects must match: {items}")
        return head

    def resolve(node, done):
        if isinstance(node, _Pending):
            return done[node.index]
        if isinstance(node, list):
            return [resolve(x, done) for x in node]
        if isinstance(node, tuple):
            return tuple(resolve(x, done) for x in node)
        if isinstance(node, dict):
            return type(node)((k, resolve(v, done)) for k, v in node.items())
        return node

    def finish(tree):
        if not groups:
            return tree
        return resolve(tree, batch_ops.concat_groups(groups))

    if all(isinstance(o, TSPipeModelOutput) for o in objs):
        return objs[0].with_data(finish(merge(*(o.data for o in objs))))
    return finish(merge(*objs))
