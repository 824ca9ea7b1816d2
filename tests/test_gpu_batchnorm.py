"""GPU parity: DeferredBatchNorm statistics, commit, normalisation and backward.

Tolerances: accumulated sums and running statistics within 1e-6 relative of an
fp64 evaluation; normalised output within 2e-5 absolute of F.batch_norm; the
state after a commit is also compared with the fp32 oracle.
"""
import pytest
import torch
import torch.nn.functional as F
from torch import nn

import tspipe_amd as ta
from helpers import max_rel_to_peak, seeded
from oracle import ts_oracle

pytestmark = pytest.mark.gpu



def _check_workspace(bn):
    # the area of the stand-alone statistics pass is left clean; of the two
    # halves that the training forward and the backward alternate between, the
    # one the NEXT call will reduce into is zero
    c = bn.num_features
    ws = bn._ws.cpu()
    assert (ws[:3 * c] == 0).all()
    nxt = 3 * c + bn._parity * 2 * c
    assert (ws[nxt:nxt + 2 * c] == 0).all()

def _rel(a, b):
    a, b = a.detach().cpu().double(), b.detach().cpu().double()
    return ((a - b).abs() / b.abs().clamp_min(1e-30)).max().item()


def _make(shape, seed, mean=0.5, std=1.5):
    return torch.randn(shape, generator=seeded(seed)) * std + mean


@pytest.mark.parametrize("shape,chunks", [((8, 16, 14, 14), 4), ((4, 7, 5, 3), 3), ((2, 3, 9), 2),
                                          ((3, 5, 2, 2, 3), 2), ((16, 64, 7, 7), 1)])
def test_deferred_bn_matches_oracle(device, shape, chunks):
    C = shape[1]
    g = seeded(40)
    gamma = torch.rand(C, generator=g) + 0.5
    beta = torch.randn(C, generator=g) * 0.1
    bn = ta.DeferredBatchNorm(C, chunks=chunks)
    with torch.no_grad():
        bn.weight.copy_(gamma)
        bn.bias.copy_(beta)
    bn = bn.to(device)
    ora = ts_oracle.DeferredBNOracle(C, chunks=chunks, weight=gamma.double(), bias=beta.double(), dtype=torch.float64)
    for step in range(2 * chunks + 1):
        x = _make(shape, 50 + step)
        y = bn(x.to(device))
        yo = ora.forward(x.double())
        assert (y.cpu().double() - yo).abs().max().item() < 2e-5
        assert bn.counter == ora.counter and bn.tracked == ora.tracked
        if ora.tracked:
            assert _rel(bn.sum, ora.sum) < 1e-6 and _rel(bn.sum_squares, ora.sum_squares) < 1e-6
        else:
            assert (bn.sum == 0).all() and (bn.sum_squares == 0).all()
        assert _rel(bn.running_mean, ora.running_mean) < 1e-6 or (ora.running_mean == 0).all()
        assert _rel(bn.running_var, ora.running_var) < 1e-6
        assert int(bn.num_batches_tracked) == int(ora.num_batches_tracked)
    _check_workspace(bn)


def test_deferred_bn_cfg5_shape(device):
    # 8 micro-batches of [32, 256, 56, 56]; oracle in fp64 on per-channel sums
    C = 256
    g = seeded(4)
    gamma = torch.rand(C, generator=g) + 0.5
    beta = torch.randn(C, generator=g) * 0.1
    bn = ta.DeferredBatchNorm(C, chunks=8)
    with torch.no_grad():
        bn.weight.copy_(gamma)
        bn.bias.copy_(beta)
    bn = bn.to(device)
    S = torch.zeros(C, dtype=torch.float64)
    Q = torch.zeros(C, dtype=torch.float64)
    cnt = 0
    for ub in range(8):
        x = torch.randn(32, C, 56, 56, generator=g) * 1.5 + 0.5
        xd = x.to(device)
        y = bn(xd)
        xs = x.double()
        S += xs.sum(dim=(0, 2, 3))
        Q += (xs * xs).sum(dim=(0, 2, 3))
        cnt += 32 * 56 * 56
        if ub in (0, 7):
            ref = F.batch_norm(xd, None, None, bn.weight, bn.bias, True, 0.0, 1e-5)
            assert (y - ref).abs().max().item() < 2e-5
            mu = xs.mean(dim=(0, 2, 3))
            var = xs.var(dim=(0, 2, 3), unbiased=False)
            want = (xs - mu[None, :, None, None]) / torch.sqrt(var + 1e-5)[None, :, None, None] \
                * gamma.double()[None, :, None, None] + beta.double()[None, :, None, None]
            assert (y.cpu().double() - want).abs().max().item() < 2e-5
        if ub == 6:
            assert _rel(bn.sum, S) < 1e-6 and _rel(bn.sum_squares, Q) < 1e-6
    mean = S / cnt
    var = Q / cnt - mean * mean  # biased
    assert _rel(bn.running_mean, 0.1 * mean) < 1e-6
    assert _rel(bn.running_var, 0.9 + 0.1 * var) < 1e-6
    assert (bn.sum == 0).all() and (bn.sum_squares == 0).all() and bn.counter == 0 and bn.tracked == 0
    assert int(bn.num_batches_tracked) == 1


def test_deferred_bn_large_mean_is_stable(device):
    # |mean| >> std: the shifted sums keep the micro-batch variance accurate
    x = torch.randn(8, 4, 32, 32, generator=seeded(41)) * 0.01 + 100.0
    bn = ta.DeferredBatchNorm(4, chunks=1, affine=False).to(device)
    y = bn(x.to(device)).cpu().double()
    xs = x.double()
    want = (xs - xs.mean(dim=(0, 2, 3), keepdim=True)) / torch.sqrt(xs.var(dim=(0, 2, 3), unbiased=False, keepdim=True) + 1e-5)
    assert (y - want).abs().max().item() < 5e-3  # fp32 input spacing at 100 is 7.6e-6, i.e. 7.6e-4 sigma
    assert _rel(bn.running_mean, 0.1 * xs.mean(dim=(0, 2, 3))) < 1e-6


def test_deferred_bn_backward(device):
    g = seeded(42)
    shape = (6, 10, 9, 7)
    x = _make(shape, 43)
    dy = torch.randn(shape, generator=g)
    bn = ta.DeferredBatchNorm(10, chunks=2).to(device)
    with torch.no_grad():
        bn.weight.copy_(torch.rand(10, generator=g) + 0.5)
        bn.bias.copy_(torch.randn(10, generator=g) * 0.1)
    xd = x.to(device).requires_grad_()
    bn(xd).backward(dy.to(device))
    x64 = x.double().requires_grad_()
    w64 = bn.weight.detach().cpu().double().requires_grad_()
    b64 = bn.bias.detach().cpu().double().requires_grad_()
    F.batch_norm(x64, None, None, w64, b64, True, 0.0, 1e-5).backward(dy.double())
    assert max_rel_to_peak(xd.grad, x64.grad) < 1e-5
    assert max_rel_to_peak(bn.weight.grad, w64.grad) < 1e-5
    assert max_rel_to_peak(bn.bias.grad, b64.grad) < 1e-5
    _check_workspace(bn)


@pytest.mark.parametrize("shape", [(2, 3, 1), (2, 5, 1, 1), (1, 2, 130, 130), (3, 4, 64, 64), (5, 3, 257),
                                   (33, 2, 7, 7), (2, 70, 3, 3), (9, 1, 4, 5), (17, 6, 2),
                                   # planes of up to 256 elements with C * HW a multiple of 4: the flat-tile kernels
                                   # (tiles that cut channels, one-element planes, a thread and a wavefront per
                                   # channel in the final sums, more than one tile and more than one slab)
                                   (64, 512, 7, 7), (37, 2048, 1, 1), (40, 24, 4, 4), (7, 36, 17), (3, 5, 16, 16),
                                   (130, 260, 3, 3), (5, 1028, 1)])
def test_deferred_bn_forward_and_backward_over_plane_and_batch_sizes(device, shape):
    # planes of one element, planes longer than one round of a wavefront's loads, planes that start off a
    # 16-byte boundary (odd sizes), more samples than a workgroup's slab, a single channel, many channels:
    # statistics, output and all three gradients against an fp64 evaluation
    C = shape[1]
    g = seeded(440 + len(shape) + shape[0])
    x = _make(shape, 441 + shape[-1])
    dy = torch.randn(shape, generator=g)
    bn = ta.DeferredBatchNorm(C, chunks=1).to(device)
    with torch.no_grad():
        bn.weight.copy_(torch.rand(C, generator=g) + 0.5)
        bn.bias.copy_(torch.randn(C, generator=g) * 0.1)
    xd = x.to(device).requires_grad_()
    y = bn(xd)
    y.backward(dy.to(device))
    x64 = x.double().requires_grad_()
    w64 = bn.weight.detach().cpu().double().requires_grad_()
    b64 = bn.bias.detach().cpu().double().requires_grad_()
    y64 = F.batch_norm(x64, None, None, w64, b64, True, 0.0, 1e-5)
    y64.backward(dy.double())
    assert (y.detach().cpu().double() - y64.detach()).abs().max().item() < 2e-5
    # dx is what is left of dy after two projections; with a handful of values per channel nearly all of
    # it cancels, so the bound is set by the size of the terms that cancel (gamma / std * |dy|), as for
    # any fp32 evaluation, and not by the size of the result
    dims_ = [0] + list(range(2, len(shape)))
    istd = 1.0 / torch.sqrt(x.double().var(dim=dims_, unbiased=False) + 1e-5)
    terms = (w64.detach().abs() * istd).max().item() * dy.abs().max().item()
    assert (xd.grad.cpu().double() - x64.grad).abs().max().item() <= 1e-5 * x64.grad.abs().max().item() + 2e-6 * terms
    n_per_channel = x.numel() // C
    assert (bn.weight.grad.cpu().double() - w64.grad).abs().max().item() \
        <= 1e-5 * w64.grad.abs().max().item() + 2e-6 * n_per_channel ** 0.5 * dy.abs().max().item()
    assert max_rel_to_peak(bn.bias.grad, b64.grad) < 1e-5
    # chunks = 1: this one micro-batch was committed (momentum 0.1, biased variance as the reference keeps it)
    dims = [0] + list(range(2, len(shape)))
    mean = x.double().mean(dim=dims)
    var = x.double().var(dim=dims, unbiased=False)
    # a mean near zero is itself a cancelled sum: bounded against the size of the values, not of the mean
    assert ((bn.running_mean.cpu().double() - 0.1 * mean).abs() <= 1e-6 * 0.1 * (mean.abs() + var.sqrt())).all()
    assert _rel(bn.running_var, 0.9 + 0.1 * var) < 1e-5
    _check_workspace(bn)


def test_deferred_bn_interleaved_forwards_and_backwards(device):
    # a pipeline runs several micro-batches forward before the first backward, and backward
    # in another order: the layer's forward and backward calls share one alternating workspace
    g = seeded(77)
    C, shape = 12, (5, 12, 8, 6)
    bn = ta.DeferredBatchNorm(C, chunks=3).to(device)
    with torch.no_grad():
        bn.weight.copy_(torch.rand(C, generator=g) + 0.5)
        bn.bias.copy_(torch.randn(C, generator=g) * 0.1)
    xs = [_make(shape, 80 + i) for i in range(3)]
    dys = [torch.randn(shape, generator=g) for _ in range(3)]
    xd = [x.to(device).requires_grad_() for x in xs]
    ys = [bn(x) for x in xd]                      # forward 0, 1, 2
    for i in (2, 0):                              # backward 2, 0
        ys[i].backward(dys[i].to(device))
    extra = bn(_make(shape, 90).to(device))       # another forward in between
    ys[1].backward(dys[1].to(device))             # backward 1
    torch.cuda.synchronize()
    w64 = bn.weight.detach().cpu().double().requires_grad_()
    b64 = bn.bias.detach().cpu().double().requires_grad_()
    for i in range(3):
        x64 = xs[i].double().requires_grad_()
        F.batch_norm(x64, None, None, w64, b64, True, 0.0, 1e-5).backward(dys[i].double())
        assert max_rel_to_peak(xd[i].grad, x64.grad) < 1e-5
    assert max_rel_to_peak(bn.weight.grad, w64.grad) < 1e-5
    assert max_rel_to_peak(bn.bias.grad, b64.grad) < 1e-5
    assert extra.shape == shape
    _check_workspace(bn)


def test_deferred_bn_eval_mode_and_momentum_none(device):
    g = seeded(44)
    bn = ta.DeferredBatchNorm(5, momentum=None, chunks=2).to(device)
    ora = ts_oracle.DeferredBNOracle(5, momentum=None, chunks=2, weight=torch.ones(5, dtype=torch.float64),
                                     bias=torch.zeros(5, dtype=torch.float64), dtype=torch.float64)
    for step in range(6):
        x = _make((4, 5, 6, 6), 60 + step)
        bn(x.to(device))
        ora.forward(x.double())
    assert int(bn.num_batches_tracked) == 3
    assert _rel(bn.running_mean, ora.running_mean) < 1e-6 and _rel(bn.running_var, ora.running_var) < 1e-6
    bn.eval()
    ora.training = False
    x = _make((3, 5, 4, 4), 70)
    xd = x.to(device).requires_grad_()
    y = bn(xd)
    assert (y.detach().cpu().double() - ora.forward(x.double())).abs().max().item() < 2e-5
    y.sum().backward()
    want = (bn.weight.detach() * torch.rsqrt(bn.running_var + bn.eps))[None, :, None, None].expand_as(x).cpu()
    assert (xd.grad.cpu() - want).abs().max().item() < 1e-5
    assert bn.tracked == 0 and bn.counter == 0  # eval does not track


def test_deferred_bn_module_contract(device):
    bn = ta.DeferredBatchNorm(4, chunks=2)
    assert set(bn.state_dict().keys()) == {"weight", "bias", "running_mean", "running_var", "num_batches_tracked",
                                           "sum", "sum_squares"}
    with pytest.raises(ValueError):
        bn.to(device)(torch.zeros(3, 4, device=device))  # 2-D input
    model = nn.Sequential(nn.Conv2d(3, 4, 3), nn.BatchNorm2d(4), nn.Sequential(nn.BatchNorm2d(4, affine=False)),
                          nn.BatchNorm2d(4, track_running_stats=False))
    conv = ta.DeferredBatchNorm.convert_deferred_batch_norm(model, chunks=3)
    assert isinstance(conv[1], ta.DeferredBatchNorm) and isinstance(conv[2][0], ta.DeferredBatchNorm)
    assert not isinstance(conv[3], ta.DeferredBatchNorm)  # no running stats: left alone
    assert conv[1].weight is model[1].weight and conv[1].running_mean is model[1].running_mean
    assert conv[1].chunks == 3 and conv[2][0].affine is False
    again = ta.DeferredBatchNorm.convert_deferred_batch_norm(conv[1], chunks=3)
    assert again is conv[1]
    conv = conv.to(device)
    out = conv(torch.randn(2, 3, 8, 8, device=device))
    assert out.shape == (2, 4, 6, 6)


def test_cpp_autograd_node_and_python_function_agree(device, monkeypatch):
    # the training forward runs from a C++ autograd node when the host helper is built, from a Python
    # autograd.Function otherwise: same launches, same bits, same bookkeeping, interleaved on one layer
    from tspipe_amd import _lib
    from tspipe_amd import batchnorm as bn_mod
    if _lib.host_helper() is None or not hasattr(_lib.host_helper(), "bn_train"):
        pytest.skip("host helper not built")
    g = seeded(610)
    results = {}
    for use_node in (True, False):
        monkeypatch.setattr(bn_mod, "_HOST_NODE", use_node)
        bn = ta.DeferredBatchNorm(12, chunks=2).to(device)
        with torch.no_grad():
            bn.weight.copy_(torch.linspace(0.5, 1.5, 12))
            bn.bias.copy_(torch.linspace(-0.2, 0.2, 12))
        outs = []
        for step in range(5):
            x = _make((6, 12, 7, 7), 620 + step).to(device).requires_grad_()
            dy = torch.randn(6, 12, 7, 7, generator=seeded(640 + step)).to(device)
            y = bn(x)
            y.backward(dy)
            outs.append((y.detach().clone(), x.grad.clone(), bn.weight.grad.clone(), bn.bias.grad.clone()))
        outs.append((bn.running_mean.clone(), bn.running_var.clone(), bn.sum.clone(), bn.sum_squares.clone()))
        _check_workspace(bn)
        assert bn.tracked == 1 and int(bn.num_batches_tracked) == 2
        results[use_node] = outs
    for a_, b_ in zip(results[True], results[False]):
        for u, v in zip(a_, b_):
            assert torch.equal(u, v)
    # the two paths on ONE layer, alternating: the shared parity keeps the workspace halves in step
    bn = ta.DeferredBatchNorm(12, chunks=1 << 30).to(device)
    for step in range(6):
        monkeypatch.setattr(bn_mod, "_HOST_NODE", step % 2 == 0)
        x = _make((6, 12, 7, 7), 660 + step).to(device).requires_grad_()
        y = bn(x)
        y.backward(torch.ones_like(y))
        want = F.batch_norm(x.detach().cpu().double(), None, None, bn.weight.detach().cpu().double(),
                            bn.bias.detach().cpu().double(), True, 0.0, 1e-5)
        assert (y.detach().cpu().double() - want).abs().max() < 2e-5
    _check_workspace(bn)
    import copy
    twin = copy.deepcopy(bn)
    assert twin._parity == bn._parity and twin._st.shared.data_ptr() != bn._st.shared.data_ptr()
    twin._parity = 1 - twin._parity
    assert twin._st.shared[0].item() == twin._parity != bn._parity


@pytest.mark.parametrize("shape", [(9, 12, 7, 7), (5, 64, 4, 4), (3, 8, 16, 16), (33, 20, 1, 1)])
def test_small_planes_flat_and_plane_kernels_agree(device, shape):
    # the same values once on a 16-byte boundary (flat-tile kernels) and once four bytes off it (the
    # wavefront-per-plane kernels): outputs, statistics and gradients agree to fp32 rounding
    from tspipe_amd import _lib
    lib = _lib.lib()
    st = torch.cuda.current_stream(device).cuda_stream
    N, C = shape[0], shape[1]
    HW = shape[2] * shape[3]
    n = N * C * HW
    g = seeded(810 + HW)
    xv = (torch.randn(n, generator=g) * 1.5 + 0.5)
    dyv = torch.randn(n, generator=g)
    gamma = (torch.rand(C, generator=g) + 0.5).to(device)
    beta = (torch.randn(C, generator=g) * 0.1).to(device)
    outs = []
    for off in (0, 1):
        buf = lambda: torch.zeros(n + 4, device=device)  # noqa: E731
        x, dy, y, dx = buf()[off:off + n], buf()[off:off + n], buf()[off:off + n], buf()[off:off + n]
        x.copy_(xv)
        dy.copy_(dyv)
        assert x.data_ptr() % 16 == 4 * off
        z = lambda k: torch.zeros(k, device=device)  # noqa: E731
        acc_s, acc_q, mean, inv, ws, dg, db = z(C), z(C), z(C), z(C), z(4 * C), z(C), z(C)
        _lib.check(lib.ts_bn_forward_train(x.data_ptr(), y.data_ptr(), gamma.data_ptr(), beta.data_ptr(), N, C, HW,
                                           acc_s.data_ptr(), acc_q.data_ptr(), mean.data_ptr(), inv.data_ptr(),
                                           ws.data_ptr(), 0, 1e-5, st), "forward")
        _lib.check(lib.ts_bn_backward(x.data_ptr(), dy.data_ptr(), mean.data_ptr(), inv.data_ptr(), gamma.data_ptr(),
                                      dx.data_ptr(), dg.data_ptr(), db.data_ptr(), ws.data_ptr(), 1, N, C, HW, 1, st),
                   "backward")
        torch.cuda.synchronize()
        assert (ws[:2 * C] == 0).all()  # the forward's half, cleared by the backward (whose own half the next call clears)
        outs.append([t.clone() for t in (y, dx, acc_s, acc_q, mean, inv, dg, db)])
    names = ("y", "dx", "sum", "sum_squares", "mean", "invstd", "dgamma", "dbeta")
    for name, a_, b_ in zip(names, *outs):
        scale = a_.abs().max().item() + 1e-12
        assert (a_ - b_).abs().max().item() <= 2e-5 * scale + 2e-6, name


def test_fused_training_forward_equals_the_two_calls(device):
    # ts_bn_forward_train against ts_bn_stats + ts_bn_apply through the C ABI: bit for bit,
    # over several calls so that both workspace halves are used and cleared
    from tspipe_amd import _lib
    lib = _lib.lib()
    st = torch.cuda.current_stream(device).cuda_stream
    N, C, H, W = 6, 10, 9, 7
    g = seeded(77)
    z = lambda n: torch.zeros(n, device=device)  # noqa: E731
    gamma, beta = torch.rand(C, generator=g).to(device) + 0.5, torch.randn(C, generator=g).to(device)
    ws2, ws4 = z(3 * C), z(4 * C)
    sum_a, sq_a, sum_b, sq_b = z(C), z(C), z(C), z(C)
    for call in range(5):
        x = (torch.randn(N, C, H, W, generator=g) * 1.5 + 0.5).to(device)
        ya, yb = torch.empty_like(x), torch.empty_like(x)
        mean_a, inv_a, mean_b, inv_b = z(C), z(C), z(C), z(C)
        _lib.check(lib.ts_bn_stats(x.data_ptr(), N, C, H * W, ws2.data_ptr(), sum_a.data_ptr(), sq_a.data_ptr(),
                                   mean_a.data_ptr(), inv_a.data_ptr(), 1e-5, st), "ts_bn_stats")
        _lib.check(lib.ts_bn_apply(x.data_ptr(), ya.data_ptr(), mean_a.data_ptr(), inv_a.data_ptr(), gamma.data_ptr(),
                                   beta.data_ptr(), N, C, H * W, 0, 1e-5, st), "ts_bn_apply")
        _lib.check(lib.ts_bn_forward_train(x.data_ptr(), yb.data_ptr(), gamma.data_ptr(), beta.data_ptr(), N, C, H * W,
                                           sum_b.data_ptr(), sq_b.data_ptr(), mean_b.data_ptr(), inv_b.data_ptr(),
                                           ws4.data_ptr(), call % 2, 1e-5, st), "ts_bn_forward_train")
        torch.cuda.synchronize()
        assert torch.equal(ya, yb)
        assert torch.equal(mean_a, mean_b) and torch.equal(inv_a, inv_b)
        assert torch.equal(sum_a, sum_b) and torch.equal(sq_a, sq_b)
        half = ws4.view(2, 2 * C)
        assert (half[1 - call % 2] == 0).all() and (half[call % 2] != 0).any()
    assert lib.ts_bn_forward_train(x.data_ptr(), yb.data_ptr(), None, None, N, C, H * W, None, None, None, None,
                                   ws4.data_ptr(), 2, 1e-5, st) == -1



def test_a_refused_call_leaves_the_next_forward_correct(device, monkeypatch):
    from tspipe_amd import _lib
    from tspipe_amd import batchnorm as bn_mod
    # the Python path is the one whose library handle can be swapped for a refusing one
    monkeypatch.setattr(bn_mod, "_HOST_NODE", False)
    bn = ta.DeferredBatchNorm(6, chunks=8).to(device)
    xs = [_make((4, 6, 5, 5), 70 + i) for i in range(3)]
    bn(xs[0].to(device))
    real = _lib.lib()

    class Refusing:
        def __getattr__(self, name):
            return getattr(real, name)

        def ts_bn_forward_train(self, *args):
            return -4  # TS_ERR_ALIGN, nothing enqueued

    parity = bn._parity
    with monkeypatch.context() as swapped:
        swapped.setattr(_lib, "lib", lambda: Refusing())
        with pytest.raises(_lib.TSPipeAmdError):
            bn(xs[1].to(device))
    assert bn._parity in (0, parity)  # not advanced by the refused call
    _check_workspace(bn)
    y = bn(xs[2].to(device))
    want = F.batch_norm(xs[2].double(), None, None, bn.weight.detach().cpu().double(), bn.bias.detach().cpu().double(),
                        True, 0.0, 1e-5)
    assert (y.cpu().double() - want).abs().max() < 2e-5
    _check_workspace(bn)
    # a cast of the module takes the workspace along; it comes back as fp32 zeros
    bn.half()
    # fp16 buffers under an fp32 input: refused on the host, before any kernel writes floats into them
    with pytest.raises(TypeError, match="fp32"):
        bn(xs[0].to(device))
    with pytest.raises(TypeError, match="fp32"):
        bn._track(xs[0].to(device))
    with pytest.raises(TypeError, match="fp32"):
        bn._commit()
    bn.float()
    assert bn._workspace(xs[0].to(device)).dtype == torch.float32
    y = bn(xs[0].to(device))
    want = F.batch_norm(xs[0].double(), None, None, bn.weight.detach().cpu().double(), bn.bias.detach().cpu().double(),
                        True, 0.0, 1e-5)
    assert (y.cpu().double() - want).abs().max() < 2e-5


@pytest.mark.parametrize("N,C,H,W", [(16, 24, 56, 56), (48, 512, 7, 7), (300, 64, 1, 1)])
def test_stand_alone_statistics_pass_is_one_launch_that_cleans_up(device, N, C, H, W):
    # ts_bn_stats with several workgroups per channel: the last one to finish does the channel's
    # bookkeeping and leaves the 3C-float workspace (sums and ticket counters) zero again; on small
    # planes (the second and third shape) a second short launch does that instead
    from tspipe_amd import _lib
    lib = _lib.lib()
    st = torch.cuda.current_stream(device).cuda_stream
    g = seeded(91)
    z = lambda n: torch.zeros(n, device=device)  # noqa: E731
    ws, acc_s, acc_q, mean, inv = z(3 * C), z(C), z(C), z(C), z(C)
    tot_s, tot_q = torch.zeros(C, dtype=torch.float64), torch.zeros(C, dtype=torch.float64)
    for call in range(3):
        x = torch.randn(N, C, H, W, generator=g) * 1.5 + 0.5
        xd = x.to(device)
        _lib.check(lib.ts_bn_stats(xd.data_ptr(), N, C, H * W, ws.data_ptr(), acc_s.data_ptr(), acc_q.data_ptr(),
                                   mean.data_ptr(), inv.data_ptr(), 1e-5, st), "ts_bn_stats")
        torch.cuda.synchronize()
        assert (ws == 0).all()
        x64 = x.double()
        tot_s += x64.sum(dim=(0, 2, 3))
        tot_q += (x64 ** 2).sum(dim=(0, 2, 3))
        m64 = x64.mean(dim=(0, 2, 3))
        v64 = x64.var(dim=(0, 2, 3), unbiased=False)
        assert _rel(acc_s, tot_s) < 1e-6 and _rel(acc_q, tot_q) < 1e-6
        assert _rel(mean, m64) < 1e-5 and _rel(inv, 1.0 / torch.sqrt(v64 + 1e-5)) < 1e-6


def test_empty_micro_batch_and_one_value_per_channel_follow_the_reference(device):
    """An empty micro-batch passes through, counts as tracked and commits 0/0 = NaN
    running statistics; one value per channel in training is tracked, committed and
    then refused as F.batch_norm refuses it (tspipe/batchnorm.py:103-120); in
    evaluation mode it is normalised like any input."""
    ref = ts_oracle.DeferredBNOracle(3, chunks=2)
    bn = ta.DeferredBatchNorm(3, chunks=2).to(device)
    g = torch.Generator().manual_seed(5)
    full = torch.randn(4, 3, 5, generator=g)
    empty = torch.randn(0, 3, 5)
    for x in (full, empty):
        want = ref.forward(x)
        got = bn(x.to(device))
        assert got.shape == want.shape
    assert bn.tracked == ref.tracked == 0 and int(bn.num_batches_tracked) == int(ref.num_batches_tracked) == 1
    # 4 x 5 values and an empty micro-batch; means near zero are sums that cancel, so the bound is on the largest
    assert max_rel_to_peak(bn.running_mean, ref.running_mean) < 1e-6
    xe = empty.to(device).requires_grad_()
    bn(xe).sum().backward()
    assert xe.grad.shape == xe.shape
    # two empty micro-batches: a commit over no values
    for _ in range(2):
        ref.forward(empty)
        bn(empty.to(device))
    assert torch.isnan(ref.running_mean).all() and torch.isnan(bn.running_mean).all()
    assert torch.isnan(ref.running_var).all() and torch.isnan(bn.running_var).all()

    ref = ts_oracle.DeferredBNOracle(3, chunks=1)
    bn = ta.DeferredBatchNorm(3, chunks=1).to(device)
    one = torch.randn(1, 3, 1, generator=g)
    with pytest.raises(ValueError, match="Expected more than 1 value per channel") as want_err:
        ref.forward(one)
    with pytest.raises(ValueError, match="Expected more than 1 value per channel") as got_err:
        bn(one.to(device))
    assert str(got_err.value) == str(want_err.value)
    assert int(bn.num_batches_tracked) == int(ref.num_batches_tracked) == 1     # tracked and committed before the refusal
    assert max_rel_to_peak(bn.running_mean, ref.running_mean) < 1e-6
    assert max_rel_to_peak(bn.running_var, ref.running_var) < 1e-6
    ref.training = False
    bn.eval()
    with torch.no_grad():
        assert (bn(one.to(device)).cpu() - ref.forward(one)).abs().max() < 2e-5
    assert bn(empty.to(device)).shape == empty.shape
