"""Pins the oracle (oracle/ts_oracle.py) without the product: each function is
checked against something that does not share its formula -- numpy fp64 closed
forms written from the mathematics, brute-force loops on tiny inputs, finite
differences, algebraic invariants and special cases with textbook answers, the
plain-C restatement, torch.nn.BatchNorm2d -- so that a dropped term, a wrong
sign or a transposed operand fails a test here."""
import ctypes
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import seeded
from oracle import ts_oracle
from tspipe_amd.shapes import numel, resnet18_shapes, vit_base_shapes

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---------------------------------------------------------------- EMA -------

def _c_oracle():
    path = os.path.join(ROOT, "oracle", "_build", "libts_oracle.so")
    if not os.path.exists(path):
        import subprocess
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True)
    return ctypes.CDLL(path)


def test_shape_lists_are_the_configs():
    r, v = resnet18_shapes(), vit_base_shapes()
    assert len(r) == 62 and sum(map(numel, r)) == 11_689_512
    assert len(v) == 152 and sum(map(numel, v)) == 86_567_656
    assert sum(1 for s in r if numel(s) <= 512) == 40  # the launch-bound tail of tiny tensors


@pytest.mark.parametrize("m", [0.996, 0.99, 0.9, 0.5, 0.0, 1.0])
def test_ema_rounding_order_c_numpy_torch_agree(m):
    g = seeded(0)
    t = torch.randn(200_003, generator=g) * 0.02
    s = torch.randn(200_003, generator=g) * 0.02
    (got,) = ts_oracle.ema_update(m, [s], [t])
    # numpy, one rounding per operation, coefficients rounded from Python doubles
    m32, c32 = np.float32(m), np.float32(1.0 - m)
    want = (t.numpy() * m32).astype(np.float32) + (s.numpy() * c32).astype(np.float32)
    assert np.array_equal(got.numpy().view(np.uint32), want.astype(np.float32).view(np.uint32))
    out = torch.empty_like(t)
    _c_oracle().ema_ref(ctypes.c_void_p(t.data_ptr()), ctypes.c_void_p(s.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                        ctypes.c_int64(t.numel()), ctypes.c_double(m))
    assert torch.equal(out.view(torch.int32), got.view(torch.int32))
    if m in (0.996, 0.99, 0.9):
        # the two plausible mistakes are visibly different from the right answer:
        fused = torch.from_numpy((t.numpy().astype(np.float64) * float(m32)
                                  + (s.numpy() * c32).astype(np.float64)).astype(np.float32))  # FMA-style single rounding
        assert (fused != got).float().mean() > 0.05
        dev_c = np.float32(1.0) - m32                                                       # 1 - m computed in fp32
        assert dev_c != c32
        wrong = torch.from_numpy((t.numpy() * m32) + (s.numpy() * dev_c))
        assert (wrong != got).float().mean() > 0.05


def test_ema_semantics():
    g = seeded(1)
    t = [torch.randn(5, 3, generator=g), torch.randn(7, generator=g), torch.randn(2, 2, generator=g)]
    s = [torch.randn(5, 3, generator=g), None, torch.randn(2, 2, generator=g)]
    t0 = [x.clone() for x in t]
    out = ts_oracle.ema_update(0.9, s, t, skip_none=True)
    assert len(out) == 2 and out[0].shape == (5, 3) and out[1].shape == (2, 2)
    assert all(torch.equal(a, b) for a, b in zip(t, t0))                    # inputs untouched
    assert all(o.data_ptr() != x.data_ptr() for o, x in zip(out, (t[0], t[2])))  # new tensors
    with pytest.raises(TypeError):
        ts_oracle.ema_update(0.9, s, t)
    same = ts_oracle.ema_update(0.996, [t[0]], [t[0]])[0]
    ulp = np.spacing(np.abs(t[0].numpy()).astype(np.float32))
    assert (np.abs(same.numpy() - t[0].numpy()) <= ulp).all()               # s == t: within one ulp
    # k iterations: t_k = m^k t_0 + (1 - m^k) s, checked in fp64
    cur, k, m = [t[0]], 50, 0.99
    for _ in range(k):
        cur = ts_oracle.ema_update(m, [s[0]], cur)
    closed = (m ** k) * t[0].double() + (1 - m ** k) * s[0].double()
    assert (cur[0].double() - closed).abs().max() < k * 2.0 ** -23 * closed.abs().max()


# ---------------------------------------------------------------- KD --------

def _kd_closed_form(s, t, T):
    """fp64 numpy: loss and d loss / d s from the definition of KL and soft-max."""
    s, t = np.asarray(s, np.float64) / T, np.asarray(t, np.float64) / T
    p = np.exp(t - t.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    q = np.exp(s - s.max(1, keepdims=True))
    q /= q.sum(1, keepdims=True)
    B = s.shape[0]
    loss = (p * (np.log(p) - np.log(q))).sum() / B * T * T
    grad = (q - p) * T / B
    return loss, grad


def test_kd_against_closed_form_bruteforce_and_finite_differences():
    g = seeded(2)
    s = torch.randn(6, 11, generator=g, dtype=torch.float64) * 3
    t = torch.randn(6, 11, generator=g, dtype=torch.float64) * 3
    T = 4.0
    sr = s.clone().requires_grad_()
    loss = ts_oracle.kd_soft_target(sr, t, T)
    loss.backward()
    want, gwant = _kd_closed_form(s.numpy(), t.numpy(), T)
    assert abs(loss.item() - want) < 1e-12 * abs(want)
    assert np.abs(sr.grad.numpy() - gwant).max() < 1e-13
    # brute force, plain Python, 3 x 5
    s3, t3 = s[:3, :5].tolist(), t[:3, :5].tolist()
    tot = 0.0
    for i in range(3):
        zs = sum(math.exp(x / T) for x in s3[i])
        zt = sum(math.exp(x / T) for x in t3[i])
        for j in range(5):
            p = math.exp(t3[i][j] / T) / zt
            q = math.exp(s3[i][j] / T) / zs
            tot += p * (math.log(p) - math.log(q))
    assert abs(ts_oracle.kd_soft_target(s[:3, :5], t[:3, :5], T).item() - tot / 3 * T * T) < 1e-12
    # central finite differences on a few coordinates
    for (i, j) in [(0, 0), (2, 7), (5, 10)]:
        e = torch.zeros_like(s)
        e[i, j] = 1e-6
        fd = (ts_oracle.kd_soft_target(s + e, t, T) - ts_oracle.kd_soft_target(s - e, t, T)).item() / 2e-6
        assert abs(fd - sr.grad[i, j].item()) < 1e-8


def test_kd_invariants():
    g = seeded(3)
    s = torch.randn(8, 20, generator=g, dtype=torch.float64) * 3
    t = torch.randn(8, 20, generator=g, dtype=torch.float64) * 3
    assert abs(ts_oracle.kd_soft_target(s, s, 4.0).item()) < 1e-15          # identical logits: zero
    base = ts_oracle.kd_soft_target(s, t, 4.0).item()
    shift = torch.randn(8, 1, generator=g, dtype=torch.float64) * 10
    assert abs(ts_oracle.kd_soft_target(s + shift, t - shift, 4.0).item() - base) < 1e-12
    assert base > 0
    sr = s.clone().requires_grad_()
    ts_oracle.kd_soft_target(sr, t, 4.0).backward()
    assert sr.grad.sum(1).abs().max() < 1e-15                                # gradient rows sum to zero
    # T -> large: T^2 * KL tends to the MSE-like limit sum((s - t - mean)^2) / (2 V B)
    big = 1e4
    d = (s - t) - (s - t).mean(1, keepdim=True)
    limit = (d * d).sum().item() / (2 * 20 * 8)
    assert abs(ts_oracle.kd_soft_target(s, t, big).item() - limit) < 1e-3 * limit


def test_distil_ce_mask_semantics():
    g = seeded(4)
    s = torch.randn(3, 5, 9, generator=g, dtype=torch.float64)
    t = torch.randn(3, 5, 9, generator=g, dtype=torch.float64)
    mask = torch.rand(3, 5, generator=g) < 0.4
    rows = mask.reshape(-1).nonzero().squeeze(1)
    want, _ = _kd_closed_form(s.reshape(-1, 9)[rows].numpy(), t.reshape(-1, 9)[rows].numpy(), 2.0)
    assert abs(ts_oracle.distil_ce(s, t, mask, 2.0, 0.5).item() - 0.5 * want) < 1e-12
    full = torch.ones(3, 5, dtype=torch.bool)
    assert abs(ts_oracle.distil_ce(s, t, full, 2.0).item()
               - ts_oracle.kd_soft_target(s.reshape(-1, 9), t.reshape(-1, 9), 2.0).item()) < 1e-12
    empty = torch.zeros(3, 5, dtype=torch.bool)
    assert torch.isnan(ts_oracle.distil_ce(s, t, empty, 2.0))               # 0/0, as in the reference
    sr = s.clone().requires_grad_()
    ts_oracle.distil_ce(sr, t, mask, 2.0).backward()
    assert (sr.grad[~mask] == 0).all() and (sr.grad[mask].abs().sum(-1) > 0).all()


# ---------------------------------------------------------------- BYOL / InfoNCE

def test_byol_special_cases_and_closed_form():
    x = torch.tensor([[3.0, 4.0, 0.0]], dtype=torch.float64)
    assert abs(ts_oracle.byol_regression_loss(x, 2.5 * x).item()) < 1e-15              # parallel
    assert abs(ts_oracle.byol_regression_loss(x, -x).item() - 4.0) < 1e-15             # opposite
    assert abs(ts_oracle.byol_regression_loss(x, torch.tensor([[0.0, 0.0, 7.0]], dtype=torch.float64)).item() - 2.0) < 1e-15
    g = seeded(5)
    o1, o2, t1, t2 = [torch.randn(9, 6, generator=g, dtype=torch.float64) for _ in range(4)]

    def cos(a, b):
        a, b = a.numpy(), b.numpy()
        return (a * b).sum(1) / np.linalg.norm(a, axis=1) / np.linalg.norm(b, axis=1)
    want = np.mean((2 - 2 * cos(o1, t2)) + (2 - 2 * cos(o2, t1)))                       # pairs are crossed
    assert abs(ts_oracle.byol_contrastive_loss(o1, o2, t1, t2).item() - want) < 1e-13
    wrong = np.mean((2 - 2 * cos(o1, t1)) + (2 - 2 * cos(o2, t2)))
    assert abs(want - wrong) > 1e-3
    r = ts_oracle.byol_regression_loss(o1, t1)
    assert ((r >= 0) & (r <= 4)).all()
    assert torch.allclose(ts_oracle.byol_regression_loss(3 * o1, 0.1 * t1), r, atol=1e-13)  # scale invariant
    a = o1.clone().requires_grad_()
    ts_oracle.byol_contrastive_loss(a, o2, t1, t2).backward()
    assert (a.grad * o1).sum(1).abs().max() < 1e-15                                       # grad orthogonal to x
    # analytic gradient: -2/N (y^ - (x^.y^) x^) / |x|
    xh, yh = F.normalize(o1, dim=1), F.normalize(t2, dim=1)
    ana = -2.0 / 9 * (yh - (xh * yh).sum(1, keepdim=True) * xh) / o1.norm(dim=1, keepdim=True)
    assert (a.grad - ana).abs().max() < 1e-14


def _infonce_closed_form(q, k, tau):
    q, k = np.asarray(q, np.float64), np.asarray(k, np.float64)
    qh = q / np.linalg.norm(q, axis=1, keepdims=True)
    kh = k / np.linalg.norm(k, axis=1, keepdims=True)
    logits = qh @ kh.T / tau
    lse = np.log(np.exp(logits - logits.max(1, keepdims=True)).sum(1)) + logits.max(1)
    n = q.shape[0]
    loss = (lse - np.diag(logits)).mean() * 2 * tau
    P = np.exp(logits - lse[:, None])
    dqh = (P - np.eye(n)) @ kh * (2.0 / n)
    dq = (dqh - qh * (qh * dqh).sum(1, keepdims=True)) / np.linalg.norm(q, axis=1, keepdims=True)
    return loss, dq


def test_infonce_against_closed_form_and_identities():
    g = seeded(6)
    q = torch.randn(8, 16, generator=g, dtype=torch.float64)
    k = torch.randn(8, 16, generator=g, dtype=torch.float64)
    qr = q.clone().requires_grad_()
    loss = ts_oracle.infonce(qr, k, 0.2)
    loss.backward()
    want, gwant = _infonce_closed_form(q.numpy(), k.numpy(), 0.2)
    assert abs(loss.item() - want) < 1e-12
    assert np.abs(qr.grad.numpy() - gwant).max() < 1e-13
    for (i, j) in [(0, 0), (3, 9), (7, 15)]:
        e = torch.zeros_like(q)
        e[i, j] = 1e-6
        fd = (ts_oracle.infonce(q + e, k, 0.2) - ts_oracle.infonce(q - e, k, 0.2)).item() / 2e-6
        assert abs(fd - qr.grad[i, j].item()) < 1e-8
    assert abs(ts_oracle.infonce(q[:1], k[:1], 0.2).item()) < 1e-15                       # N = 1
    assert abs(ts_oracle.infonce(3 * q, 0.5 * k, 0.2).item() - loss.item()) < 1e-12       # scale invariant
    assert (qr.grad * q).sum(1).abs().max() < 1e-15                                       # rows orthogonal to q
    # transposing the logits (k as queries) gives a different loss: the operand order is pinned
    assert abs(ts_oracle.infonce(k, q, 0.2).item() - loss.item()) > 1e-4
    # k == q unit vectors and tiny tau: the diagonal dominates, loss -> 0
    u = F.normalize(q, dim=1)
    assert ts_oracle.infonce(u, u, 0.01).item() < 1e-8
    # both directions are summed by the pair form, with crossed views
    o1, o2, t1, t2 = q, k, torch.randn(8, 16, generator=g, dtype=torch.float64), torch.randn(8, 16, generator=g, dtype=torch.float64)
    pair = ts_oracle.moco_contrastive_loss(o1, o2, t1, t2, 0.2).item()
    a, _ = _infonce_closed_form(o1.numpy(), t2.numpy(), 0.2)
    b, _ = _infonce_closed_form(o2.numpy(), t1.numpy(), 0.2)
    assert abs(pair - (a + b)) < 1e-12


# ---------------------------------------------------------------- DeferredBatchNorm

def test_deferred_bn_oracle_against_fp64_sums():
    g = seeded(7)
    C, chunks = 5, 3
    gamma = (torch.rand(C, generator=g) + 0.5).double()
    beta = (torch.randn(C, generator=g) * 0.1).double()
    bn = ts_oracle.DeferredBNOracle(C, chunks=chunks, weight=gamma, bias=beta, dtype=torch.float64)
    xs = [(torch.randn(4, C, 3, 2, generator=g) * 1.5 + 0.5).double() for _ in range(chunks)]
    for i, x in enumerate(xs):
        y = bn.forward(x)
        mu = x.mean(dim=(0, 2, 3), keepdim=True)
        var = ((x - mu) ** 2).mean(dim=(0, 2, 3), keepdim=True)                      # this micro-batch's own, biased
        want = (x - mu) / torch.sqrt(var + 1e-5) * gamma.view(1, C, 1, 1) + beta.view(1, C, 1, 1)
        assert (y - want).abs().max() < 1e-12
        if i < chunks - 1:
            assert bn.tracked == i + 1 and bn.counter == (i + 1) * 4 * 6
            allx = torch.cat(xs[:i + 1])
            assert (bn.sum - allx.sum(dim=(0, 2, 3))).abs().max() < 1e-12
            assert (bn.sum_squares - (allx ** 2).sum(dim=(0, 2, 3))).abs().max() < 1e-11
            assert (bn.running_mean == 0).all() and (bn.running_var == 1).all()      # deferred: nothing committed yet
    allx = torch.cat(xs)
    mean = allx.mean(dim=(0, 2, 3))
    var_b = allx.var(dim=(0, 2, 3), unbiased=False)
    assert (bn.running_mean - 0.1 * mean).abs().max() < 1e-13
    assert (bn.running_var - (0.9 + 0.1 * var_b)).abs().max() < 1e-12                # biased variance
    assert bn.tracked == 0 and bn.counter == 0 and (bn.sum == 0).all() and (bn.sum_squares == 0).all()
    assert int(bn.num_batches_tracked) == 1


def test_deferred_bn_oracle_vs_nn_batchnorm_and_modes():
    g = seeded(8)
    x = (torch.randn(6, 4, 5, 5, generator=g) * 2 + 1).double()
    n = 6 * 25
    ref = torch.nn.BatchNorm2d(4).double()
    ref.train()
    y_ref = ref(x)
    bn = ts_oracle.DeferredBNOracle(4, chunks=1, weight=torch.ones(4, dtype=torch.float64),
                                    bias=torch.zeros(4, dtype=torch.float64), dtype=torch.float64)
    y = bn.forward(x)
    assert (y - y_ref).abs().max() < 1e-12
    assert (bn.running_mean - ref.running_mean).abs().max() < 1e-14                  # chunks=1: same running mean
    new_ref = (ref.running_var - 0.9) / 0.1                                           # unbiased batch variance
    new_bn = (bn.running_var - 0.9) / 0.1
    assert (new_bn - new_ref * (n - 1) / n).abs().max() < 1e-12                       # biased = (n-1)/n * unbiased
    bn.training = False
    ref.eval()
    ref.running_var.copy_(bn.running_var)
    x2 = (torch.randn(2, 4, 3, 3, generator=g)).double()
    assert (bn.forward(x2) - ref(x2)).abs().max() < 1e-13                             # eval: affine map of running stats
    assert bn.tracked == 0
    with pytest.raises(ValueError):
        bn.forward(torch.zeros(3, 4, dtype=torch.float64))
    # momentum=None: cumulative average with factor 1/num_batches_tracked
    cm = ts_oracle.DeferredBNOracle(4, momentum=None, chunks=1, dtype=torch.float64)
    means = []
    for i in range(3):
        xi = (torch.randn(3, 4, 2, 2, generator=g) + i).double()
        cm.forward(xi)
        means.append(xi.mean(dim=(0, 2, 3)))
    # factor 1/k makes running_mean the plain average of the batch means (the initial 0 is wiped by factor 1)
    assert (cm.running_mean - torch.stack(means).mean(0)).abs().max() < 1e-13


# ---------------------------------------------------------------- scatter / gather

def test_scatter_gather_oracle_identities():
    g = seeded(9)
    for n, k in [(5, 4), (6, 4), (1, 4), (3, 8), (32, 4), (7, 1)]:
        x = torch.randn(n, 3, generator=g)
        pieces = ts_oracle.scatter(x, k)
        size = -(-n // k)
        assert [p.shape[0] for p in pieces] == [min(size, n - i) for i in range(0, n, size)]  # ceil(N/k) rule
        assert torch.equal(ts_oracle.gather(pieces), x)
    a, b = torch.randn(6, 2, generator=g), torch.randint(0, 9, (6,), generator=g)
    back = ts_oracle.gather(ts_oracle.scatter((a, b), 4))
    assert torch.equal(back[0], a) and torch.equal(back[1], b)
    # byte concatenation in C agrees with torch.cat
    pieces = [torch.randn(r, 5, generator=g) for r in (2, 0, 3)]
    want = torch.cat(pieces)
    out = torch.empty_like(want)
    ptrs = (ctypes.c_void_p * 3)(*[p.data_ptr() for p in pieces])
    sizes = (ctypes.c_int64 * 3)(*[p.numel() * 4 for p in pieces])
    _c_oracle().cat_ref(ptrs, sizes, ctypes.c_int64(3), ctypes.c_void_p(out.data_ptr()))
    assert torch.equal(out, want)


# ---------------------------------------------------------------- combined distillation losses

def test_soft_target_tspipe_loss_closed_form():
    g = seeded(10)
    s = torch.randn(7, 9, generator=g, dtype=torch.float64) * 2
    t = torch.randn(7, 9, generator=g, dtype=torch.float64) * 2
    y = torch.randint(0, 9, (7,), generator=g)
    kd, gkd = _kd_closed_form(s.numpy(), t.numpy(), 4.0)
    sn = s.numpy()
    lse = np.log(np.exp(sn - sn.max(1, keepdims=True)).sum(1)) + sn.max(1)
    ce = (lse - sn[np.arange(7), y.numpy()]).mean()
    sr = s.clone().requires_grad_()
    loss = ts_oracle.soft_target_tspipe_loss(sr, t, y, 4.0, 0.7)
    loss.backward()
    assert abs(loss.item() - (ce + 0.7 * kd)) < 1e-12
    soft = np.exp(sn - lse[:, None])
    onehot = np.eye(9)[y.numpy()]
    assert np.abs(sr.grad.numpy() - (0.7 * gkd + (soft - onehot) / 7)).max() < 1e-13


def test_distil_loss_terms_use_their_own_row_sets():
    g = seeded(11)
    bs, seq, V, H = 2, 5, 11, 6
    s = torch.randn(bs, seq, V, generator=g, dtype=torch.float64)
    t = torch.randn(bs, seq, V, generator=g, dtype=torch.float64)
    sh = torch.randn(bs, seq, H, generator=g, dtype=torch.float64)
    th = torch.randn(bs, seq, H, generator=g, dtype=torch.float64)
    lm = torch.full((bs, seq), -100, dtype=torch.long)
    lm[0, 1], lm[1, 3], lm[1, 4] = 3, 0, 10
    att = torch.tensor([[1, 1, 1, 0, 0], [1, 1, 1, 1, 1]], dtype=torch.bool)
    for restrict in (True, False):
        got = ts_oracle.distil_loss(s, t, sh, th, lm, att, 0.5, 2.0, 1.5, 2.0, restrict).item()
        kd_rows = (lm.reshape(-1) > -1) if restrict else att.reshape(-1)
        kd, _ = _kd_closed_form(s.reshape(-1, V)[kd_rows].numpy(), t.reshape(-1, V)[kd_rows].numpy(), 2.0)
        ce_rows = lm.reshape(-1) != -100
        sn = s.reshape(-1, V)[ce_rows].numpy()
        lab = lm.reshape(-1)[ce_rows].numpy()
        lse = np.log(np.exp(sn).sum(1))
        ce = (lse - sn[np.arange(len(lab)), lab]).mean()
        a, b = sh.reshape(-1, H)[att.reshape(-1)].numpy(), th.reshape(-1, H)[att.reshape(-1)].numpy()
        cos = (a * b).sum(1) / np.sqrt(((a * a).sum(1) + 1e-12) * ((b * b).sum(1) + 1e-12))
        want = 0.5 * kd + 2.0 * ce + 1.5 * (1 - cos).mean()
        assert abs(got - want) < 1e-12


def test_logits_mse_and_kd_mode_logits_closed_form():
    g = seeded(12)
    s = torch.randn(6, 10, generator=g, dtype=torch.float64) * 2
    t = torch.randn(6, 10, generator=g, dtype=torch.float64) * 2
    y = torch.randint(0, 10, (6,), generator=g)
    sn, tn = s.numpy(), t.numpy()
    assert abs(ts_oracle.logits_mse(s, t).item() - ((sn - tn) ** 2).mean()) < 1e-14
    lse = np.log(np.exp(sn).sum(1))
    ce = (lse - sn[np.arange(6), y.numpy()]).mean()
    sr = s.clone().requires_grad_()
    loss = ts_oracle.soft_target_tspipe_loss(sr, t, y, 4.0, 0.3, kd_mode="logits")
    loss.backward()
    assert abs(loss.item() - (ce + 0.3 * ((sn - tn) ** 2).mean())) < 1e-12
    soft = np.exp(sn - lse[:, None])
    want = (soft - np.eye(10)[y.numpy()]) / 6 + 0.3 * 2 * (sn - tn) / 60
    assert np.abs(sr.grad.numpy() - want).max() < 1e-13
    # the teacher gets no gradient
    tr = t.clone().requires_grad_()
    assert not ts_oracle.soft_target_tspipe_loss(s, tr, y, 4.0, 0.3, kd_mode="logits").requires_grad


def test_distil_loss_clm_and_mse_terms_closed_form():
    g = seeded(13)
    bs, seq, V = 2, 5, 7
    s = torch.randn(bs, seq, V, generator=g, dtype=torch.float64)
    t = torch.randn(bs, seq, V, generator=g, dtype=torch.float64)
    lm = torch.full((bs, seq), -100, dtype=torch.long)
    lm[0, 0], lm[0, 2], lm[1, 4], lm[1, 1] = 5, 3, 6, 0
    att = torch.tensor([[1, 1, 1, 1, 0], [1, 1, 0, 0, 0]], dtype=torch.bool)
    sn, tn = s.numpy(), t.numpy()
    lse = np.log(np.exp(sn).sum(-1))
    for restrict in (True, False):
        rows = ((lm > -1) if restrict else att).numpy()
        kd, _ = _kd_closed_form(sn[rows], tn[rows], 2.0)
        base = ts_oracle.distil_loss(s, t, None, None, lm, att, 0.5, 0.0, 0.0, 2.0, restrict).item()
        assert abs(base - 0.5 * kd) < 1e-12
        # causal LM: the logits at position p are scored against the label at p+1.
        # Labelled positions: (0,0)->p=-1 (none), (0,2)->p=1, (1,4)->p=3, (1,1)->p=0
        clm_terms = [lse[0, 1] - sn[0, 1, 3], lse[1, 3] - sn[1, 3, 6], lse[1, 0] - sn[1, 0, 0]]
        got = ts_oracle.distil_loss(s, t, None, None, lm, att, 0.5, 0.0, 0.0, 2.0, restrict, alpha_clm=1.5).item()
        assert abs(got - (0.5 * kd + 1.5 * np.mean(clm_terms))) < 1e-12
        # squared error: summed over the selected rows, divided by their number (not by elements)
        mse = ((sn[rows] - tn[rows]) ** 2).sum() / rows.sum()
        got = ts_oracle.distil_loss(s, t, None, None, lm, att, 0.5, 0.0, 0.0, 2.0, restrict, alpha_mse=0.25).item()
        assert abs(got - (0.5 * kd + 0.25 * mse)) < 1e-12

