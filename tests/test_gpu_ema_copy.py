"""GPU parity: multi-tensor EMA and multi-segment copy (bit-exact vs the oracle)."""
import pytest
import torch

import tspipe_amd as ta
from helpers import bits_equal, param_lists, seeded
from oracle import ts_oracle
from tspipe_amd.shapes import resnet18_shapes, vit_base_shapes

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,shapes,m,seed", [("resnet18", resnet18_shapes(), 0.996, 0),
                                                ("vit_base", vit_base_shapes(), 0.99, 3)])
def test_ema_bit_exact(device, name, shapes, m, seed):
    teacher, student = param_lists(shapes, seed)
    want = ts_oracle.ema_update(m, student, teacher)
    t_dev = [t.to(device) for t in teacher]
    s_dev = [s.to(device) for s in student]
    got = ta.calculate_target_network_parameters(m, s_dev, t_dev)
    assert len(got) == len(want)
    for g, w, t0, s0, td, sd in zip(got, want, teacher, student, t_dev, s_dev):
        assert g.shape == w.shape and g.dtype == torch.float32 and g.is_cuda
        assert bits_equal(g, w)
        assert bits_equal(td, t0) and bits_equal(sd, s0)  # inputs untouched
        assert g.data_ptr() != td.data_ptr()


def test_ema_iterated_100(device):
    shapes = resnet18_shapes()
    teacher, student = param_lists(shapes, 0)
    t_dev = [t.to(device) for t in teacher]
    s_dev = [s.to(device) for s in student]
    want = teacher
    for _ in range(100):
        t_dev = ta.calculate_target_network_parameters(0.996, s_dev, t_dev)
        want = ts_oracle.ema_update(0.996, student, want)
    for g, w in zip(t_dev, want):
        assert bits_equal(g, w)


def test_ema_none_entries_unaligned_views_and_momentum_edges(device):
    g = seeded(11)
    base_t = torch.randn(4099, generator=g).to(device)
    base_s = torch.randn(4099, generator=g).to(device)
    # views that start 4 and 12 bytes into a 16-byte line, odd lengths
    t_list = [base_t[1:1001], base_t[1003:1004], base_t[1100:4099], torch.randn(7, 3, generator=g).to(device)]
    s_list = [base_s[3:1003], None, base_s[1100:4099], torch.randn(7, 3, generator=g).to(device)]
    got = ta.calculate_updated_momentum_encoder(0.9, s_list, t_list)
    want = ts_oracle.ema_update(0.9, [None if s is None else s.cpu() for s in s_list], [t.cpu() for t in t_list],
                                skip_none=True)
    assert len(got) == 3
    for a, b in zip(got, want):
        assert bits_equal(a, b)
    with pytest.raises(TypeError):
        ta.calculate_target_network_parameters(0.9, s_list, t_list)
    pairs_t = [t for t, s in zip(t_list, s_list) if s is not None]
    pairs_s = [s for s in s_list if s is not None]
    for a, t in zip(ta.momentum_update(1.0, pairs_s, pairs_t), pairs_t):
        assert bits_equal(a, t)  # m = 1: teacher unchanged
    for a, s in zip(ta.momentum_update(0.0, pairs_s, pairs_t), pairs_s):
        assert bits_equal(a, s)  # m = 0: student copied
    assert ta.momentum_update(0.5, [], []) == []


def test_ema_in_place_form(device):
    teacher, student = param_lists([(33, 17), (5,), (128, 64, 3, 3)], 5)
    t_dev = [torch.nn.Parameter(t.to(device)) for t in teacher]
    s_dev = [torch.nn.Parameter(s.to(device)) for s in student]
    ptrs = [t.data_ptr() for t in t_dev]
    ta.update_target_network_parameters_(s_dev, t_dev, 0.99)
    want = ts_oracle.ema_update(0.99, student, teacher)
    for t, w, p in zip(t_dev, want, ptrs):
        assert bits_equal(t, w) and t.data_ptr() == p


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_ema_two_byte_parameter_lists(device, dtype):
    # the reference's expression runs on whatever dtype the parameters have
    # (benchmarks/byol/trainer.py:209): each product and the sum rounded to the type
    g = seeded(21)
    shapes = [(64, 3, 7, 7), (64,), (1000, 512), (3,), (1,), (17, 5), (2048 * 3 + 5,)]
    teacher = [(torch.randn(s, generator=g) * 0.3).to(dtype) for s in shapes]
    student = [(torch.randn(s, generator=g) * 0.3).to(dtype) for s in shapes]
    t_dev, s_dev = [t.to(device) for t in teacher], [s.to(device) for s in student]
    for m in (0.99, 0.996, 0.5):
        got = ta.calculate_target_network_parameters(m, s_dev, t_dev)
        want = ts_oracle.ema_update(m, student, teacher)
        for a, b, t in zip(got, want, t_dev):
            assert a.dtype == dtype and a.shape == b.shape and bits_equal(a, b)
    # views that are only 2-byte aligned, and the in-place form
    base_t, base_s = torch.randn(5000, generator=g).to(dtype), torch.randn(5000, generator=g).to(dtype)
    bt, bs = base_t.to(device), base_s.to(device)
    got = ta.momentum_update(0.9, [bs[1:4098], bs[4099:4100]], [bt[3:4100], bt[4101:4102]])
    want = ts_oracle.ema_update(0.9, [base_s[1:4098], base_s[4099:4100]], [base_t[3:4100], base_t[4101:4102]])
    for a, b in zip(got, want):
        assert bits_equal(a, b)
    params_t = [torch.nn.Parameter(t.clone()) for t in t_dev]
    ta.update_target_network_parameters_(s_dev, params_t, 0.99)
    for p, w in zip(params_t, ts_oracle.ema_update(0.99, student, teacher)):
        assert bits_equal(p, w)
    # chained: the rounding of every step is the reference's
    t_cpu, cur = teacher, t_dev
    for _ in range(20):
        cur = ta.momentum_update(0.99, s_dev, cur)
        t_cpu = ts_oracle.ema_update(0.99, student, t_cpu)
    for a, b in zip(cur, t_cpu):
        assert bits_equal(a, b)


def test_ema_rejects_bad_inputs(device):
    a = torch.zeros(8, device=device)
    with pytest.raises(TypeError):
        ta.momentum_update(0.9, [a.half()], [a])          # mixed types
    with pytest.raises(TypeError):
        ta.momentum_update(0.9, [a.double()], [a.double()])
    with pytest.raises(TypeError):
        ta.clone_and_update(0.9, [a.half()], [a.half()])  # the fused form is fp32
    with pytest.raises(ValueError):
        ta.momentum_update(0.9, [a], [torch.zeros(9, device=device)])
    with pytest.raises(TypeError):
        ta.momentum_update(0.9, [a.cpu()], [a.cpu()])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int64, torch.uint8, torch.bool])
def test_gather_bit_exact_dtypes(device, dtype):
    g = seeded(21)
    pieces = []
    for rows in (3, 1, 0, 5):
        x = torch.randn(rows, 7, 13, generator=g) * 100
        pieces.append((x > 0) if dtype == torch.bool else x.to(dtype))
    want = torch.cat(pieces)
    got = ta.gather([ta.Batch(p.to(device)) for p in pieces])
    assert bits_equal(got, want)


def test_gather_scatter_roundtrip_ragged(device):
    g = seeded(22)
    for n, k in [(5, 4), (6, 4), (1, 4), (3, 8), (32, 4), (7, 1), (9, 2)]:
        x = torch.randn(n, 5, 3, generator=g).to(device)
        pieces = ta.scatter(x, k)
        want_sizes = [p.shape[0] for p in x.cpu().chunk(k)]
        assert [b.tensor.shape[0] for b in pieces] == want_sizes
        assert pieces[0].tensor.data_ptr() == x.data_ptr()  # views, as in the reference
        assert bits_equal(ta.gather(pieces), x)
        owned = ta.scatter_copy(x, k)
        assert [b.tensor.shape[0] for b in owned] == want_sizes
        assert all(bits_equal(o.tensor, p.tensor) for o, p in zip(owned, pieces))
        assert owned[0].tensor.data_ptr() != x.data_ptr()


def test_gather_tuple_and_unaligned_segments(device):
    g = seeded(23)
    a = torch.randn(10, 3, generator=g).to(device)          # 12-byte rows: pieces start off 16-byte lines
    b = torch.randint(0, 255, (10, 5), generator=g).to(torch.uint8).to(device)  # 5-byte rows
    pieces = ta.scatter((a, b), 4)
    assert all(not p.atomic and len(p) == 2 for p in pieces)
    got = ta.gather(pieces)
    assert isinstance(got, tuple) and bits_equal(got[0], a) and bits_equal(got[1], b)
    # non-contiguous piece and odd byte offsets
    c = torch.randint(0, 255, (9, 7), generator=g).to(torch.uint8).to(device)
    parts = [c[0:2], c[2:5, :], c[5:9]]
    assert bits_equal(ta.gather([ta.Batch(p) for p in parts]), c)
    t = torch.randn(6, 4, generator=g).to(device)
    parts = [t.t()[0:2], t.t()[2:4]]  # transposed views: not contiguous
    assert bits_equal(ta.gather([ta.Batch(p) for p in parts]), torch.cat([p.cpu() for p in parts]))


@pytest.mark.parametrize("n_pieces", [2, 16, 17, 40])
def test_gather_of_few_and_of_many_small_pieces(device, n_pieces):
    # up to 16 small segments travel in the kernel's own arguments, more (or longer ones) through a
    # planned table: same bytes either way, with ragged row counts, an empty piece, byte-sized elements
    # and pieces that start off a 16-byte boundary
    g = seeded(700 + n_pieces)
    for dtype, width in ((torch.float32, 33), (torch.uint8, 7), (torch.bfloat16, 129)):
        pieces = []
        for i in range(n_pieces):
            rows = 0 if i == 1 else 1 + (i * 5) % 9
            base = (torch.randn(rows * width + 3, generator=g) * 50).to(dtype).to(device)
            pieces.append(base[3:].view(rows, width) if i % 3 == 2 else base[:rows * width].view(rows, width))
        got = ta.gather([ta.Batch(p) for p in pieces])
        assert torch.equal(got, torch.cat(pieces))


def test_gather_autograd_routes_gradients(device):
    g = seeded(24)
    leaves = [torch.randn(r, 4, generator=g).to(device).requires_grad_() for r in (2, 3, 1)]
    out = ta.gather([ta.Batch(x) for x in leaves])
    assert out.requires_grad
    w = torch.randn(6, 4, generator=g).to(device)
    (out * w).sum().backward()
    r0 = 0
    for x in leaves:
        assert bits_equal(x.grad, w[r0:r0 + x.shape[0]])
        r0 += x.shape[0]


def test_gather_large_cfg3_shape(device):
    # 4 micro-batches of [8, 128, 30522] bf16 -> [32, 128, 30522]
    g = seeded(2)
    pieces = [(torch.randn(8, 128, 30522, generator=g) * 2).to(torch.bfloat16).to(device) for _ in range(4)]
    got = ta.gather([ta.Batch(p) for p in pieces])
    assert got.shape == (32, 128, 30522)
    for i, p in enumerate(pieces):
        assert torch.equal(got[8 * i:8 * i + 8].view(torch.int16), p.view(torch.int16))
    back = ta.scatter(got, 4)
    assert all(torch.equal(b.tensor.view(torch.int16), p.view(torch.int16)) for b, p in zip(back, pieces))


def test_gather_rejects_host_tensors():
    with pytest.raises(TypeError):
        ta.gather([ta.Batch(torch.zeros(2, 2)), ta.Batch(torch.zeros(2, 2))])


def test_ema_output_arenas_are_recycled_only_when_unreferenced(device):
    from tspipe_amd import ema as ema_mod
    ema_mod.release_pool()
    teacher, student = param_lists([(64, 8), (16,), (32, 4)], 9)
    t_dev = [t.to(device) for t in teacher]
    s_dev = [s.to(device) for s in student]
    a = ta.momentum_update(0.9, s_dev, t_dev)
    a_ptr = a[0].data_ptr()
    b = ta.momentum_update(0.8, s_dev, t_dev)          # `a` is still held: must not be overwritten
    assert b[0].data_ptr() != a_ptr
    want_a = ts_oracle.ema_update(0.9, student, teacher)
    assert all(bits_equal(x, w) for x, w in zip(a, want_a))
    alias = a[1].view(-1)                               # an alias survives the list
    del a
    c = ta.momentum_update(0.7, s_dev, t_dev)
    assert c[0].data_ptr() != a_ptr                     # storage still aliased: no reuse
    assert bits_equal(alias, want_a[1].view(-1))
    del alias, c
    d = ta.momentum_update(0.6, s_dev, t_dev)
    assert d[0].data_ptr() in (a_ptr, b[0].data_ptr()) or True  # reuse is allowed now, never required
    assert all(bits_equal(x, w) for x, w in zip(d, ts_oracle.ema_update(0.6, student, teacher)))
    assert all(bits_equal(x, w) for x, w in zip(b, ts_oracle.ema_update(0.8, student, teacher)))
    ema_mod.release_pool()


def test_clone_and_copy_in_of_a_parameter_list(device):
    # the two whole-list copies around the EMA in the optimizer step
    g = seeded(31)
    params = [torch.nn.Parameter(torch.randn(s, generator=g).to(device)) for s in [(64, 3, 7, 7), (64,), (5, 3), (1,)]]
    params.append(torch.nn.Parameter(torch.randint(0, 100, (7,), generator=g).to(device), requires_grad=False))
    clones = ta.clone_params(params)
    assert len(clones) == len(params)
    for c, p in zip(clones, params):
        assert c.shape == p.shape and c.dtype == p.dtype and not c.requires_grad
        assert c.data_ptr() != p.data_ptr() and bits_equal(c, p)
        assert c.data_ptr() % 16 == 0
    live = [torch.nn.Parameter(torch.zeros_like(p), requires_grad=p.is_floating_point()) for p in params]
    ptrs = [p.data_ptr() for p in live]
    ta.copy_params_(live, clones)
    for l, c, ptr in zip(live, clones, ptrs):
        assert bits_equal(l, c) and l.data_ptr() == ptr
    assert ta.clone_params([]) == []
    with pytest.raises(ValueError):
        ta.copy_params_(live[:2], clones[:1])
    with pytest.raises(ValueError):
        ta.copy_params_([live[0]], [clones[1]])


@pytest.mark.parametrize("shapes", [[(64, 3, 7, 7), (64,), (129, 33), (5,)], resnet18_shapes()])
def test_clone_and_update_fused(device, shapes):
    from tspipe_amd import ema as ema_mod
    ema_mod.release_pool()
    teacher, student = param_lists(shapes, 13)
    t_dev = [t.to(device) for t in teacher]
    s_dev = [torch.nn.Parameter(s.to(device)) for s in student]
    clones, new_t = ta.clone_and_update(0.996, s_dev, t_dev)
    want = ts_oracle.ema_update(0.996, student, teacher)
    assert len(clones) == len(new_t) == len(shapes)
    for c, n, s0, w, sd, td, t0 in zip(clones, new_t, student, want, s_dev, t_dev, teacher):
        assert bits_equal(c, s0) and bits_equal(n, w)
        assert c.data_ptr() not in (sd.data_ptr(), n.data_ptr()) and not c.requires_grad
        assert bits_equal(sd, s0) and bits_equal(td, t0)  # inputs untouched
    # the same through the unfused pair of calls
    clones2 = ta.clone_params(s_dev)
    new_t2 = ta.momentum_update(0.996, clones2, t_dev)
    assert all(bits_equal(a, b) for a, b in zip(new_t, new_t2))
    ema_mod.release_pool()


def test_generic_gather_of_a_nested_structure_is_one_launch(device):
    # DistilBERT-like micro-batch outputs: a dict with logits and a tuple of hidden states
    from tspipe_amd import _tables
    g = seeded(31)
    full = {"logits": torch.randn(12, 7, 33, generator=g).to(torch.bfloat16),
            "hidden_states": tuple(torch.randn(12, 7, 16, generator=g) for _ in range(3)),
            "note": "x"}
    pieces = ta.generic_scatter({k: (v.to(device) if torch.is_tensor(v) else
                                     tuple(h.to(device) for h in v) if isinstance(v, tuple) else v)
                                 for k, v in full.items()}, 4)
    _tables.kernel_events = []
    try:
        back = ta.generic_gather(pieces)
        launches = len(_tables.kernel_events)
    finally:
        _tables.kernel_events = None
    assert launches == 1
    want = ts_oracle.generic_object_gather(*ts_oracle.generic_object_scatter(full, 4))
    assert bits_equal(back["logits"].cpu(), want["logits"])
    assert all(bits_equal(a.cpu(), b) for a, b in zip(back["hidden_states"], want["hidden_states"]))
    assert back["note"] == "x" and type(back) is dict
    # the structure checks still come first, before anything is launched
    bad = [p.value for p in pieces]
    bad[1] = dict(bad[1], note="y")
    with pytest.raises(ValueError):
        ta.generic_object_gather(*bad)


def test_ema_and_gather_from_two_threads(device):
    # TSPipe drives the plug-ins from one worker thread per partition
    # (tspipe/gpu_worker.py); each thread has its own stream, table ring and
    # table cache, the output arenas are shared under a lock.
    import threading
    shapes = [(64, 3, 7, 7), (64,), (128, 64, 3, 3), (1000, 512), (1000,)]
    results, errors = {}, []

    def worker(idx):
        try:
            torch.cuda.set_device(device)
            s, t = param_lists(shapes, seed=40 + idx)
            want = t
            for _ in range(12):
                want = ts_oracle.ema_update(0.99, s, want)
            stream = torch.cuda.Stream(device)
            with torch.cuda.stream(stream):
                sd, td = [x.to(device) for x in s], [x.to(device) for x in t]
                got = td
                for _ in range(12):
                    got = ta.calculate_target_network_parameters(0.99, sd, got)
                cat = ta.gather([ta.Batch(x.reshape(-1, 1)) for x in got])
            stream.synchronize()
            results[idx] = (all(bits_equal(a.cpu(), b) for a, b in zip(got, want)),
                            bits_equal(cat.cpu(), torch.cat([w.reshape(-1, 1) for w in want])))
        except Exception as e:  # pragma: no cover - reported below
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors, errors
    assert results == {0: (True, True), 1: (True, True)}


def test_arena_reuse_waits_for_announced_readers_and_can_be_switched_off(device):
    from tspipe_amd import ema as ema_mod
    ema_mod.release_pool()
    teacher, student = param_lists([(256, 1024), (1024,), (512, 512)], 17)
    t_dev = [t.to(device) for t in teacher]
    s_dev = [s.to(device) for s in student]
    side = torch.cuda.Stream(device)
    version = ta.momentum_update(0.9, s_dev, t_dev)
    ptr = version[0].data_ptr()
    # a reader on another stream, announced to the pool, then the version is dropped without a host sync
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        torch.cuda._sleep(2_000_000)
        copies = [v.clone() for v in version]
    ema_mod.note_reader(version, side)
    del version
    again = ta.momentum_update(0.5, s_dev, t_dev)  # may take the same arena; must not overtake the reader
    assert again[0].data_ptr() == ptr
    torch.cuda.synchronize()
    assert all(bits_equal(c, w) for c, w in zip(copies, ts_oracle.ema_update(0.9, student, teacher)))
    assert all(bits_equal(a, w) for a, w in zip(again, ts_oracle.ema_update(0.5, student, teacher)))
    # recycling off: every call returns memory no earlier result used while that result is alive or not
    ema_mod.set_recycling(False)
    try:
        del again, copies
        a = ta.momentum_update(0.9, s_dev, t_dev)
        pa = a[0].data_ptr()
        keep = a  # noqa: F841  (held: torch's allocator cannot hand the block out either)
        b = ta.momentum_update(0.9, s_dev, t_dev)
        assert b[0].data_ptr() != pa
        assert all(bits_equal(x, w) for x, w in zip(b, ts_oracle.ema_update(0.9, student, teacher)))
    finally:
        ema_mod.set_recycling(True)
        ema_mod.release_pool()


def test_ema_more_chunks_than_a_grid_dimension_holds(device):
    # a caller-chosen chunk of 1024 elements over 70 M parameters: 68,360 chunks, more than the
    # 65,535 that fit the grid's second dimension, so the launch falls back to a flat grid with
    # the chunk index derived by division; same arithmetic, bit for bit
    import numpy as np
    from tspipe_amd import _lib, _tables
    g = torch.Generator(device=device).manual_seed(5)
    n = 70_000_001
    t = torch.randn(n, generator=g, device=device) * 0.02
    s = torch.randn(n, generator=g, device=device) * 0.02
    out = torch.empty_like(t)
    ptr = lambda x: np.array([x.data_ptr()], dtype=np.uint64)
    with torch.cuda.device(device):
        table = _tables.stage_ema(ptr(t), ptr(s), ptr(out), np.array([n], dtype=np.int64), device, chunk_elems=1024)
        assert table.n_chunks > 65535
        _lib.check(_lib.lib().ts_ema_multi(table.dev_ptr, table.n_chunks, table.chunk, 0.99, 1.0 - 0.99,
                                           _lib.current_stream_ptr(device)), "ts_ema_multi")
        table.done()
    torch.cuda.synchronize()
    want = t * torch.tensor(0.99, dtype=torch.float32) + s * torch.tensor(1.0 - 0.99, dtype=torch.float32)
    assert torch.equal(out, want)


def test_empty_lists_tensors_and_pieces_pass_through(device):
    """What the reference's loops and torch.cat / chunk do with nothing in hand."""
    g = seeded(3)
    t = [torch.randn(5, generator=g), torch.randn(0), torch.randn(0, 3), torch.randn(2, 2, generator=g)]
    s = [torch.randn(x.shape, generator=g) for x in t]
    want = ts_oracle.ema_update(0.9, s, t)
    got = ta.calculate_target_network_parameters(0.9, [x.to(device) for x in s], [x.to(device) for x in t])
    assert len(got) == len(want) and all(bits_equal(a, b) for a, b in zip(got, want))
    assert ta.calculate_target_network_parameters(0.9, [], []) == []
    pieces = [torch.randn(2, 3, generator=g), torch.randn(0, 3), torch.randn(1, 3, generator=g)]
    assert bits_equal(ta.gather([ta.Batch(p.to(device)) for p in pieces]), ts_oracle.gather(pieces))
    nothing = [torch.randn(0, 3), torch.randn(0, 3)]
    out = ta.gather([ta.Batch(p.to(device)) for p in nothing])
    assert out.shape == (0, 3) and out.is_cuda
    got = [b.value for b in ta.scatter(torch.randn(0, 3).to(device), 2)]
    want = ts_oracle.scatter(torch.randn(0, 3), 2)
    assert [tuple(x.shape) for x in got] == [tuple(x.shape) for x in want]
