"""Host-side logic (no GPU): Batch, scatter, the structure-aware scatter/gather,
TSPipeModelWrapper -- replayed against fixtures recorded from the reference
(tests/golden/structure_cases.json) and against the oracle's restatement.

Tensor concatenation itself is device-only in the product; here the leaf
concatenation is swapped for torch.cat so that the *structure* handling can be
exercised on CPU tensors.  The device path is covered by the GPU tests.
"""
import pickle
from collections import OrderedDict

import pytest
import torch

import tspipe_amd as ta
from oracle import ts_oracle
from structure_util import attempt, build, load_cases, run_batch_op
from tspipe_amd import batch_ops

CASES = load_cases()
OUT, BATCH = ta.TSPipeModelOutput, ta.Batch


@pytest.fixture
def cpu_cat(monkeypatch):
    monkeypatch.setattr(batch_ops, "concat_dim0", lambda pieces: torch.cat(tuple(pieces)))
    monkeypatch.setattr(batch_ops, "concat_groups", lambda groups: [torch.cat(tuple(g)) for g in groups])


@pytest.mark.parametrize("case", CASES["generic_scatter"], ids=lambda c: str(c["input"])[:40])
def test_generic_scatter_matches_reference_fixture(case):
    got = attempt(lambda: ta.generic_object_scatter(build(case["input"], OUT), case["chunks"]), OUT, BATCH)
    assert got == case["result"]
    # and the oracle's restatement agrees with the fixture too
    ora = attempt(lambda: ts_oracle.generic_object_scatter(build(case["input"], OUT), case["chunks"], output_cls=OUT),
                  OUT, BATCH)
    assert ora == case["result"]


@pytest.mark.parametrize("case", CASES["generic_gather"], ids=lambda c: str(c["inputs"])[:40])
def test_generic_gather_matches_reference_fixture(case, cpu_cat):
    objs = lambda: [build(r, OUT) for r in case["inputs"]]  # noqa: E731
    got = attempt(lambda: ta.generic_object_gather(*objs()), OUT, BATCH)
    assert got == case["result"]
    ora = attempt(lambda: ts_oracle.generic_object_gather(*objs(), output_cls=OUT), OUT, BATCH)
    assert ora == case["result"]


@pytest.mark.parametrize("case", CASES["scatter_gather"], ids=lambda c: str(c["input"])[:40])
def test_scatter_gather_matches_reference_fixture(case, cpu_cat):
    got = attempt(lambda: ta.scatter(build(case["input"], OUT), case["chunks"]), OUT, BATCH)
    assert got == case["scatter"]
    back = attempt(lambda: ta.gather(ta.scatter(build(case["input"], OUT), case["chunks"])), OUT, BATCH)
    assert back == case["roundtrip"]


@pytest.mark.parametrize("case", CASES["batch"], ids=lambda c: f"{c['op']}-{str(c['input'])[:20]}")
def test_batch_container_matches_reference_fixture(case):
    got = attempt(lambda: run_batch_op(ta.Batch, build(case["input"], OUT), case["op"], case["args"]), OUT, BATCH)
    assert got == case["result"]


def test_scatter_returns_views_and_follows_chunk_rule():
    for n, k in [(5, 4), (6, 4), (1, 4), (3, 8), (32, 4), (0, 3)]:
        x = torch.arange(n * 3, dtype=torch.float32).reshape(n, 3)
        pieces = ta.scatter(x, k)
        want = x.chunk(k)
        assert [tuple(p.tensor.shape) for p in pieces] == [tuple(w.shape) for w in want]
        for p, w in zip(pieces, want):
            assert p.tensor.data_ptr() == w.data_ptr()  # a view of the input, like the reference
            assert torch.equal(p.tensor, w)
        assert [tuple(o.shape) for o in ts_oracle.scatter(x, k)] == [tuple(w.shape) for w in want]
    # tuple input: position-aligned, truncated to the member with the fewest chunks
    a, b = torch.zeros(5, 2), torch.zeros(8)
    pieces = ta.scatter((a, b), 4)
    assert len(pieces) == 3 and all(len(p) == 2 for p in pieces)


def test_generic_scatter_gather_roundtrip_values(cpu_cat):
    x = {"logits": torch.arange(24.).reshape(6, 4), "hidden_states": (torch.arange(12.).reshape(6, 2),), "n": 3}
    pieces = ta.generic_scatter(x, 3)
    assert all(isinstance(p, ta.Batch) and not p.atomic for p in pieces)
    back = ta.generic_gather(pieces)
    assert torch.equal(back["logits"], x["logits"]) and torch.equal(back["hidden_states"][0], x["hidden_states"][0])
    assert back["n"] == 3
    od = OrderedDict(a=torch.zeros(4, 1))
    assert type(ta.generic_object_scatter(od, 2)[0]) is dict  # OrderedDict in, plain dict pieces out
    t = torch.arange(6.).reshape(6, 1)
    assert torch.equal(ta.generic_gather(ta.generic_scatter(t, 4)), t)


def test_batch_transforms_and_check():
    b = ta.Batch((torch.ones(2, requires_grad=True), torch.zeros(3)))
    c = b.clone()
    assert not c.atomic and c[0].data_ptr() != b[0].data_ptr() and torch.equal(c[0], b[0])
    d = b.detach()
    assert not d[0].requires_grad
    assert [t.shape for t in b] == [torch.Size([2]), torch.Size([3])]
    doubled = ta.Batch(torch.ones(2)).call(lambda t: t * 2)
    assert doubled.atomic and torch.equal(doubled.tensor, torch.full((2,), 2.))
    assert ta.Batch(torch.ones(2)).to_(torch.device("cpu")).tensor.device.type == "cpu"
    assert "atomic=True" in repr(ta.Batch(torch.ones(1)))
    ta.check(torch.ones(1))
    ta.check((torch.ones(1), (torch.ones(2),)))
    with pytest.raises(TypeError):
        ta.check([torch.ones(1)])
    with pytest.raises(TypeError):
        ta.check((torch.ones(1), 3))
    assert ta.batch_size(torch.zeros(7, 2)) == 7
    with pytest.raises(NotImplementedError):
        ta.batch_size({"x": torch.zeros(1)})
    fn = ta.defaultScatterGatherFn
    assert fn.scatter is ta.scatter and fn.gather is ta.gather and fn.batch_size is ta.batch_size


def test_traverse_tensor_map_keeps_structure():
    obj = {"a": [torch.ones(2), (torch.zeros(1), 5)], "b": OrderedDict(x=torch.ones(3)), "c": "s"}
    out = ta.traverse_tensor_map(obj, lambda t: t + 1)
    assert torch.equal(out["a"][0], torch.full((2,), 2.)) and out["a"][1][1] == 5 and out["c"] == "s"
    assert isinstance(out["b"], OrderedDict) and isinstance(out["a"][1], tuple)
    wrapped = ta.TSPipeModelOutput(data=obj, lst_require_grad_tensor_path=[("a", 0)])
    out = ta.traverse_tensor_map(wrapped, lambda t: t * 0)
    assert isinstance(out, ta.TSPipeModelOutput) and out.lst_require_grad_tensor_path == [("a", 0)]
    assert out.data["b"]["x"].sum() == 0


def test_model_wrapper_contract():
    class Plain(torch.nn.Module):
        def forward(self, x):
            return x * 2

    class Rich(torch.nn.Module):
        def forward(self, x):
            return {"logits": x["ids"].float(), "hidden_states": (x["ids"],)}

    w = ta.TSPipeModelWrapper(Plain())
    y = w(torch.ones(2))
    assert torch.is_tensor(y) and torch.equal(y, torch.full((2,), 2.))
    y = w(ta.TSPipeModelOutput(data=torch.ones(2), lst_require_grad_tensor_path=None))  # unwraps its input
    assert torch.is_tensor(y)
    r = ta.TSPipeModelWrapper(Rich())({"ids": torch.arange(3)})
    assert isinstance(r, ta.TSPipeModelOutput) and r.lst_require_grad_tensor_path is None
    assert set(r.data.keys()) == {"logits", "hidden_states"}


def test_plugins_are_picklable_module_level_objects():
    # TSPipe pickles its plug-ins into spawned workers (tspipe/gpu_worker.py:596-600)
    for obj in (ta.calculate_target_network_parameters, ta.calculate_updated_momentum_encoder,
                ta.byol_contrastive_loss, ta.moco_contrastive_loss, ta.defaultScatterGatherFn,
                ta.ScatterGatherFn(ta.generic_scatter, ta.generic_gather, ta.batch_size), ta.SoftTarget(4.0),
                ta.DeferredBatchNorm(4, chunks=2), ta.TSPipeModelOutput(data=1, lst_require_grad_tensor_path=None)):
        clone = pickle.loads(pickle.dumps(obj))
        assert type(clone) is type(obj)


def test_product_refuses_host_tensors():
    with pytest.raises(TypeError):
        ta.gather([ta.Batch(torch.zeros(2, 2)), ta.Batch(torch.zeros(2, 2))])
    with pytest.raises(TypeError):
        ta.momentum_update(0.9, [torch.zeros(4)], [torch.zeros(4)])
    with pytest.raises(TypeError):
        ta.SoftTarget(4.0)(torch.zeros(2, 3), torch.zeros(2, 3))
    with pytest.raises(TypeError):
        ta.byol_loss(*[torch.zeros(2, 3)] * 4)
    with pytest.raises(TypeError):
        ta.infonce_loss(torch.zeros(2, 64), torch.zeros(2, 64), 0.2)
    with pytest.raises(TypeError):
        ta.DeferredBatchNorm(3)(torch.zeros(2, 3, 4))
    with pytest.raises(ValueError):
        ta.DeferredBatchNorm(3)(torch.zeros(2, 3))  # fewer than 3 dims: the reference's own check


def test_bind_params_repoints_without_copy():
    import tspipe_amd as ta
    model = torch.nn.Sequential(torch.nn.Linear(4, 3), torch.nn.Linear(3, 2))
    params = list(model.parameters())
    ids = [id(p) for p in params]
    version = [torch.randn_like(p) for p in params]
    ta.bind_params_(model.parameters(), version)
    assert [id(p) for p in model.parameters()] == ids          # same Parameter objects
    for p, v in zip(model.parameters(), version):
        assert p.data_ptr() == v.data_ptr() and p.requires_grad  # aliasing the version, still trainable leaves
        assert torch.equal(p, v)
    x = torch.randn(5, 4)
    want = torch.nn.functional.linear(torch.nn.functional.linear(x, version[0], version[1]), version[2], version[3])
    assert torch.equal(model(x), want)
    with pytest.raises(ValueError):
        ta.bind_params_(model.parameters(), version[:-1])
    with pytest.raises(ValueError):
        ta.bind_params_(model.parameters(), [v.double() for v in version])



def test_deferred_bn_refuses_cast_state_on_the_host():
    # module.half() casts the accumulators, running statistics and affine parameters; the kernels
    # read and write C floats, so the mismatch is an error raised before anything is launched
    bn = ta.DeferredBatchNorm(4, chunks=2)
    x = torch.zeros(2, 4, 3, 3)
    bn._require_state(x)
    bn.half()
    with pytest.raises(TypeError, match="sum is torch.float16"):
        bn._require_state(x)
    bn.float()
    bn.weight.data = bn.weight.data.double()
    with pytest.raises(TypeError, match="weight is torch.float64"):
        bn._require_state(x)
