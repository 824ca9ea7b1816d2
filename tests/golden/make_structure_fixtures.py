"""Writes tests/golden/structure_cases.json: how the reference's own
generic_object_scatter / generic_object_gather / scatter / gather / Batch treat
odd structures (types, lengths, shapes of what comes back; exceptions raised).

Run once in the build container, where the reference is mounted at
/root/reference; the JSON it writes is the committed fixture.  Inputs are
described by small recipes so that the test can rebuild them without the
reference.  Only structure is recorded (container types, tensor shapes,
exception class names), never tensor values: the values are pinned bit-exactly
against torch.chunk / torch.cat elsewhere.
"""
import json
import os
import sys
from collections import OrderedDict

import torch

sys.path.insert(0, "/root/reference")
from tspipe.batch_ops import Batch, gather, scatter  # noqa: E402
from tspipe.model_wrapper import TSPipeModelOutput  # noqa: E402
from tspipe.utils import generic_object_gather, generic_object_scatter  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def build(recipe):
    """recipe -> object.  ["T", d0, d1..] tensor of that shape (arange values);
    ["list", ...], ["tuple", ...], ["dict", [k, v]...], ["odict", ...], ["out", r] TSPipeModelOutput;
    ["lit", x] a plain Python value."""
    kind = recipe[0]
    if kind == "T":
        shape = recipe[1:]
        n = 1
        for s in shape:
            n *= s
        return torch.arange(n, dtype=torch.float32).reshape(shape)
    if kind == "list":
        return [build(r) for r in recipe[1:]]
    if kind == "tuple":
        return tuple(build(r) for r in recipe[1:])
    if kind == "dict":
        return {k: build(v) for k, v in recipe[1:]}
    if kind == "odict":
        return OrderedDict((k, build(v)) for k, v in recipe[1:])
    if kind == "out":
        return TSPipeModelOutput(data=build(recipe[1]), lst_require_grad_tensor_path=[("logits",)])
    if kind == "lit":
        return recipe[1]
    raise ValueError(kind)


def describe(o):
    if isinstance(o, torch.Tensor):
        return {"tensor": list(o.shape)}
    if isinstance(o, TSPipeModelOutput):
        return {"out": describe(o.data), "paths": [list(p) for p in (o.lst_require_grad_tensor_path or [])]}
    if isinstance(o, Batch):
        return {"batch": describe(o.value), "atomic": bool(o.atomic)}
    if isinstance(o, OrderedDict):
        return {"odict": [[k, describe(v)] for k, v in o.items()]}
    if isinstance(o, dict):
        return {"dict": [[k, describe(v)] for k, v in o.items()]}
    if isinstance(o, list):
        return {"list": [describe(v) for v in o]}
    if isinstance(o, (tuple, zip)):
        return {"tuple": [describe(v) for v in o]}
    return {"lit": o}


def attempt(fn):
    try:
        return {"ok": describe(fn())}
    except Exception as e:  # noqa: BLE001
        return {"raises": type(e).__name__}


SCATTER_CASES = [
    (["T", 8, 3], 4), (["T", 5, 2], 4), (["T", 6], 4), (["T", 1, 2], 4), (["T", 3, 2], 8),
    (["tuple", ["T", 8, 3], ["T", 8]], 4), (["tuple", ["T", 5, 3], ["T", 8]], 4),
    (["list", ["T", 4, 2], ["lit", 7]], 2), (["list", ["T", 5, 2], ["lit", "x"]], 4),
    (["dict", ["logits", ["T", 8, 5]], ["hidden_states", ["tuple", ["T", 8, 2], ["T", 8, 3]]]], 4),
    (["odict", ["a", ["T", 4, 2]], ["b", ["lit", None]]], 2),
    (["dict", ["a", ["T", 3, 2]], ["b", ["lit", 1.5]]], 4),
    (["out", ["dict", ["logits", ["T", 6, 4]], ["n", ["lit", 3]]]], 3),
    (["lit", 5], 3), (["tuple"], 2), (["list"], 2), (["dict"], 2),
    (["list", ["list", ["T", 4, 1], ["T", 4, 2]], ["tuple", ["T", 4]]], 2),
]

GATHER_CASES = [
    [["T", 2, 3], ["T", 3, 3]],
    [["tuple", ["T", 2, 3], ["T", 2]], ["tuple", ["T", 1, 3], ["T", 1]]],
    [["list", ["T", 2, 1], ["lit", 7]], ["list", ["T", 2, 1], ["lit", 7]]],
    [["list", ["T", 2, 1], ["lit", 7]], ["list", ["T", 2, 1], ["lit", 8]]],
    [["dict", ["a", ["T", 2, 2]]], ["dict", ["a", ["T", 1, 2]]]],
    [["dict", ["a", ["T", 2, 2]]], ["dict", ["b", ["T", 1, 2]]]],
    [["odict", ["a", ["T", 2, 2]]], ["odict", ["a", ["T", 1, 2]]]],
    [["dict", ["a", ["T", 2, 2]]], ["odict", ["a", ["T", 1, 2]]]],
    [["list", ["T", 2]], ["tuple", ["T", 2]]],
    [["out", ["dict", ["logits", ["T", 2, 4]]]], ["out", ["dict", ["logits", ["T", 3, 4]]]]],
    [["lit", 3], ["lit", 3]], [["lit", 3], ["lit", 4]],
    [["T", 2, 3], ["T", 2, 4]],
    [],
]

BATCH_OPS = [
    # (recipe, op name, args)
    (["T", 4, 2], "getitem", [0]), (["T", 4, 2], "getitem", [1]),
    (["tuple", ["T", 4], ["T", 4, 2]], "getitem", [1]),
    (["T", 4, 2], "len", []), (["tuple", ["T", 4], ["T", 4, 2]], "len", []),
    (["T", 4, 2], "tensor", []), (["T", 4, 2], "tensors", []),
    (["tuple", ["T", 4]], "tensor", []), (["tuple", ["T", 4]], "tensors", []),
    (["T", 4, 2], "setitem_int", [0]), (["T", 4, 2], "setitem_int", [1]),
    (["tuple", ["T", 4], ["T", 4, 2]], "setitem_int", [1]),
    (["T", 4, 2], "setitem_slice_all_1", []), (["T", 4, 2], "setitem_slice_all_2", []),
    (["tuple", ["T", 4], ["T", 4, 2]], "setitem_slice_all_2", []),
    (["T", 4, 2], "setitem_slice_partial", []),
]


def run_batch_op(recipe, op, args):
    b = Batch(build(recipe))
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


def main():
    out = {"generic_scatter": [], "generic_gather": [], "scatter_gather": [], "batch": []}
    for recipe, chunks in SCATTER_CASES:
        out["generic_scatter"].append({"input": recipe, "chunks": chunks,
                                       "result": attempt(lambda: generic_object_scatter(build(recipe), chunks))})
    for recipes in GATHER_CASES:
        out["generic_gather"].append({"inputs": recipes,
                                      "result": attempt(lambda: generic_object_gather(*[build(r) for r in recipes]))})
    for recipe, chunks in SCATTER_CASES[:7]:
        res = attempt(lambda: scatter(build(recipe), chunks))
        back = attempt(lambda: gather(scatter(build(recipe), chunks)))
        out["scatter_gather"].append({"input": recipe, "chunks": chunks, "scatter": res, "roundtrip": back})
    for recipe, op, args in BATCH_OPS:
        out["batch"].append({"input": recipe, "op": op, "args": args,
                             "result": attempt(lambda: run_batch_op(recipe, op, args))})
    with open(os.path.join(HERE, "structure_cases.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print("wrote", len(out["generic_scatter"]), len(out["generic_gather"]), len(out["scatter_gather"]), len(out["batch"]))


if __name__ == "__main__":
    main()
