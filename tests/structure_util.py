"""Rebuilds the inputs of tests/golden/structure_cases.json and describes results
in the fixture's vocabulary (container kinds, tensor shapes, exception names)."""
import json
import os
from collections import OrderedDict

import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def load_cases():
    with open(os.path.join(HERE, "golden", "structure_cases.json")) as f:
        return json.load(f)


def build(recipe, output_cls, device="cpu"):
    kind = recipe[0]
    if kind == "T":
        shape = recipe[1:]
        n = 1
        for s in shape:
            n *= s
        return torch.arange(n, dtype=torch.float32, device=device).reshape(shape)
    if kind == "list":
        return [build(r, output_cls, device) for r in recipe[1:]]
    if kind == "tuple":
        return tuple(build(r, output_cls, device) for r in recipe[1:])
    if kind == "dict":
        return {k: build(v, output_cls, device) for k, v in recipe[1:]}
    if kind == "odict":
        return OrderedDict((k, build(v, output_cls, device)) for k, v in recipe[1:])
    if kind == "out":
        return output_cls(data=build(recipe[1], output_cls, device), lst_require_grad_tensor_path=[("logits",)])
    if kind == "lit":
        return recipe[1]
    raise ValueError(kind)


def describe(o, output_cls, batch_cls):
    if isinstance(o, torch.Tensor):
        return {"tensor": list(o.shape)}
    if isinstance(o, output_cls):
        return {"out": describe(o.data, output_cls, batch_cls),
                "paths": [list(p) for p in (o.lst_require_grad_tensor_path or [])]}
    if isinstance(o, batch_cls):
        return {"batch": describe(o.value, output_cls, batch_cls), "atomic": bool(o.atomic)}
    if isinstance(o, OrderedDict):
        return {"odict": [[k, describe(v, output_cls, batch_cls)] for k, v in o.items()]}
    if isinstance(o, dict):
        return {"dict": [[k, describe(v, output_cls, batch_cls)] for k, v in o.items()]}
    if isinstance(o, list):
        return {"list": [describe(v, output_cls, batch_cls) for v in o]}
    if isinstance(o, (tuple, zip)):
        return {"tuple": [describe(v, output_cls, batch_cls) for v in o]}
    return {"lit": o}


def attempt(fn, output_cls, batch_cls):
    try:
        return {"ok": describe(fn(), output_cls, batch_cls)}
    except Exception as e:  # noqa: BLE001
        return {"raises": type(e).__name__}


def run_batch_op(batch_cls, value, op, args):
    b = batch_cls(value)
    new = torch.zeros(9)
    if op == "getitem":
        return b[args[0]]
    if op == "len":
        return len(b)
    if op == "tensor":
        return b.tensor
    if op == "tensors":
        return b.tensors
    if op == "setitem_int":
        b[args[0]] = new
        return b
    if op == "setitem_slice_all_1":
        b[:] = (new,)
        return b
    if op == "setitem_slice_all_2":
        b[:] = (new, new)
        return b
    if op == "setitem_slice_partial":
        b[0:1] = (new,)
        return b
    raise ValueError(op)
