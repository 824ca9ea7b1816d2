"""GPU parity: KD soft target (plain and masked), BYOL and InfoNCE losses against the oracle.

Tolerances.  fp32 inputs: loss and gradient within 1e-5 (relative for the
loss, max-abs over the gradient's peak for the gradient) of the fp64 oracle.
bf16 inputs: the oracle is evaluated in fp64 on the same bf16 values; loss
within 1e-3 relative, gradient within 1e-3 of the gradient's peak plus the
bf16 rounding of the stored gradient itself (2^-9 relative per element).
"""
import pytest
import torch

import tspipe_amd as ta
from helpers import bits_equal, max_rel_to_peak, rel_err, seeded
from oracle import ts_oracle

pytestmark = pytest.mark.gpu


def _oracle_grad(fn, *student, others=()):
    xs = [s.detach().double().requires_grad_() for s in student]
    loss = fn(*xs, *[o.double() for o in others])
    loss.backward()
    return loss.item(), [x.grad for x in xs]


def test_kd_cfg2_fp32(device):
    g = seeded(1)
    s = torch.randn(256, 100, generator=g) * 3
    t = torch.randn(256, 100, generator=g) * 3
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.kd_soft_target(a, b, 4.0), s, others=(t,))
    sd = s.to(device).requires_grad_()
    loss = ta.SoftTarget(4.0)(sd, t.to(device))
    loss.backward()
    assert loss.dtype == torch.float32 and loss.dim() == 0
    assert rel_err(loss.item(), want) < 1e-5
    assert max_rel_to_peak(sd.grad, gw) < 1e-5
    # against the fp32 eager chain too (the reference's own arithmetic)
    s32 = s.clone().requires_grad_()
    l32 = ts_oracle.kd_soft_target(s32, t, 4.0)
    l32.backward()
    assert rel_err(loss.item(), l32.item()) < 1e-5
    assert max_rel_to_peak(sd.grad, s32.grad) < 1e-5


@pytest.mark.parametrize("rows,V", [(1, 1), (3, 5), (7, 63), (5, 64), (4, 65), (9, 1000), (2, 2049), (3, 4099),
                                    (5, 8191), (2, 16380), (2, 16381), (2, 32760), (2, 32761)])
def test_kd_shapes_fp32(device, rows, V):
    g = seeded(100 + V)
    s = torch.randn(rows, V, generator=g) * 3
    t = torch.randn(rows, V, generator=g) * 3
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.kd_soft_target(a, b, 2.5), s, others=(t,))
    sd = s.to(device).requires_grad_()
    loss = ta.kd_soft_target_loss(sd, t.to(device), 2.5)
    loss.backward()
    assert rel_err(loss.item(), want) < 2e-5 or abs(loss.item() - want) < 1e-7
    assert max_rel_to_peak(sd.grad, gw) < 2e-5 or gw.abs().max() < 1e-12


@pytest.mark.parametrize("rows,V", [(5, 4097), (4, 9001), (3, 30522), (2, 32760), (2, 32761), (3, 50257), (2, 65520),
                                    (2, 65521)])
def test_kd_long_rows_bf16_unmasked(device, rows, V):
    # rows of 8 K to 64 K bf16 logits without a mask: one launch with the row pair in registers
    # (512 threads per row up to 32760 elements, 1024 up to 65520, here also with rows that start
    # off a 16-byte boundary), two passes beyond
    g = seeded(300 + V)
    s = (torch.randn(rows, V, generator=g) * 2).to(torch.bfloat16)
    t = (torch.randn(rows, V, generator=g) * 2).to(torch.bfloat16)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.kd_soft_target(a, b, 2.0), s, others=(t,))
    sd = s.to(device).requires_grad_()
    loss = ta.kd_soft_target_loss(sd, t.to(device), 2.0)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-3
    err = (sd.grad.cpu().double() - gw).abs()
    assert (err <= 1e-3 * gw.abs().max() + gw.abs() * 2.0 ** -8).all()


def test_kd_long_rows_operands_aligned_differently(device):
    # student and teacher rows at different offsets from a 16-byte boundary: same results
    # as for aligned operands (the kernels fall back to element-wise access where they must)
    g = seeded(41)
    rows, V = 3, 6000
    s = torch.randn(rows, V, generator=g) * 3
    t = torch.randn(rows, V, generator=g) * 3
    ref_s = s.to(device).requires_grad_()
    ref = ta.kd_soft_target_loss(ref_s, t.to(device), 3.0)
    ref.backward()
    pad = torch.zeros(rows * V + 1, device=device)
    pad[1:] = s.to(device).reshape(-1)
    shifted = pad[1:].view(rows, V).detach().requires_grad_()  # data pointer 4 bytes past a 16-byte boundary
    assert shifted.data_ptr() % 16 == 4 and shifted.is_contiguous()
    got = ta.kd_soft_target_loss(shifted, t.to(device), 3.0)
    got.backward()
    assert rel_err(got.item(), ref.item()) < 1e-6
    assert max_rel_to_peak(shifted.grad, ref_s.grad.cpu()) < 1e-6


def test_kd_identities(device):
    g = seeded(7)
    s = (torch.randn(16, 50, generator=g) * 3).to(device)
    same = s.clone().requires_grad_()
    loss = ta.kd_soft_target_loss(same, s, 4.0)
    loss.backward()
    assert abs(loss.item()) < 1e-6 and same.grad.abs().max().item() < 1e-7  # s == t
    t = (torch.randn(16, 50, generator=g) * 3).to(device)
    a = s.clone().requires_grad_()
    l1 = ta.kd_soft_target_loss(a, t, 4.0)
    l1.backward()
    shift = torch.randn(16, 1, generator=g).to(device) * 10
    b = (s + shift).requires_grad_()
    l2 = ta.kd_soft_target_loss(b, t - shift, 4.0)
    l2.backward()
    assert rel_err(l2.item(), l1.item()) < 1e-4  # per-row constants cancel
    assert (a.grad - b.grad).abs().max().item() < 1e-6
    assert a.grad.sum(dim=1).abs().max().item() < 1e-6  # gradient rows sum to zero
    assert l1.item() >= 0


@pytest.mark.parametrize("rows,V,dtype", [(6, 100, torch.float32), (4, 1000, torch.float32), (3, 30522, torch.bfloat16),
                                          (2, 70001, torch.float32)])
def test_kd_teacher_minus_inf_entries_contribute_nothing(device, rows, V, dtype):
    # a masked vocabulary: the teacher puts -inf on some entries, the student's are finite.
    # F.kl_div's xlogy gives those entries a zero term; a plain 0 * (-inf) would be NaN
    g = seeded(300 + V)
    s = (torch.randn(rows, V, generator=g) * 3).to(dtype)
    t = (torch.randn(rows, V, generator=g) * 3).to(dtype)
    banned = torch.rand(rows, V, generator=g) < 0.3
    banned[:, 0] = False  # no row is banned entirely
    t = t.masked_fill(banned, float("-inf"))
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.kd_soft_target(a, b, 2.0), s, others=(t,))
    assert want == want  # the reference's value is finite
    sd = s.to(device).requires_grad_()
    loss = ta.kd_soft_target_loss(sd, t.to(device), 2.0)
    loss.backward()
    tol = 2e-5 if dtype == torch.float32 else 1e-3
    assert rel_err(loss.item(), want) < tol
    assert torch.isfinite(sd.grad).all()
    assert max_rel_to_peak(sd.grad, gw) < tol + (0 if dtype == torch.float32 else 2 ** -8)


def test_kd_grad_output_scaling_and_no_grad(device):
    g = seeded(8)
    s = (torch.randn(8, 33, generator=g)).to(device)
    t = (torch.randn(8, 33, generator=g)).to(device)
    a = s.clone().requires_grad_()
    ta.kd_soft_target_loss(a, t, 2.0).backward()
    b = s.clone().requires_grad_()
    (ta.kd_soft_target_loss(b, t, 2.0) * 3.0).backward()
    assert torch.allclose(b.grad, 3.0 * a.grad, rtol=1e-6, atol=0)
    c = s.clone().requires_grad_()
    ta.kd_soft_target_loss(c, t, 2.0, weight=3.0).backward()
    assert torch.allclose(c.grad, b.grad, rtol=1e-5, atol=1e-9)
    with torch.no_grad():
        l = ta.kd_soft_target_loss(s, t, 2.0)
    assert not l.requires_grad


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_kd_masked_wide_vocab_half(device, dtype):
    # DistilBERT-shaped rows (vocab 30522: rows are not 16-byte aligned), fewer rows than cfg3
    g = seeded(2)
    bs, seq, V = 4, 32, 30522
    s = (torch.randn(bs, seq, V, generator=g) * 2).to(dtype)
    t = (torch.randn(bs, seq, V, generator=g) * 2).to(dtype)
    mask = torch.rand(bs, seq, generator=g) < 0.15
    assert 0 < mask.sum().item() < bs * seq
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.distil_ce(a, b, mask, 2.0, 0.5), s, others=(t,))
    sd = s.to(device).requires_grad_()
    loss = ta.distil_ce_loss(sd, t.to(device), mask.to(device), 2.0, 0.5)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-3
    peak = gw.abs().max().item()
    err = (sd.grad.cpu().double() - gw).abs()
    assert (err <= 1e-3 * peak + gw.abs() * 2.0 ** -8).all()
    assert sd.grad.dtype == dtype and sd.grad.shape == s.shape
    unsel = ~mask
    assert (sd.grad.cpu()[unsel] == 0).all()  # dense gradient, zero outside the mask


def test_kd_mask_special_cases(device):
    g = seeded(3)
    s = (torch.randn(2, 6, 40, generator=g) * 2)
    t = (torch.randn(2, 6, 40, generator=g) * 2)
    sd, td = s.to(device), t.to(device)
    full = torch.ones(2, 6, dtype=torch.bool)
    a = ta.distil_ce_loss(sd, td, full.to(device), 2.0).item()
    b = ta.kd_soft_target_loss(sd.view(-1, 40), td.view(-1, 40), 2.0).item()
    assert rel_err(a, b) < 1e-6  # all-true mask == unmasked over all rows
    one = torch.zeros(2, 6, dtype=torch.bool)
    one[1, 2] = True
    want = ts_oracle.distil_ce(s.double(), t.double(), one, 2.0).item()
    assert rel_err(ta.distil_ce_loss(sd, td, one.to(device), 2.0).item(), want) < 1e-5
    none = torch.zeros(2, 6, dtype=torch.bool)
    x = sd.clone().requires_grad_()
    l = ta.distil_ce_loss(x, td, none.to(device), 2.0)
    l.backward()
    assert torch.isnan(l).item() and torch.isnan(ts_oracle.distil_ce(s, t, none, 2.0)).item()  # 0/0 like the reference
    assert (x.grad == 0).all()
    # integer attention mask is accepted like a bool one
    att = torch.tensor([[1, 1, 0, 0, 1, 0], [0, 1, 1, 1, 0, 0]])
    want = ts_oracle.distil_ce(s.double(), t.double(), att.bool(), 2.0).item()
    assert rel_err(ta.distil_ce_loss(sd, td, att.to(device), 2.0).item(), want) < 1e-5


@pytest.mark.parametrize("V,dtype", [(9001, torch.bfloat16), (40000, torch.bfloat16), (5000, torch.float32)])
def test_kd_mask_special_cases_long_rows(device, V, dtype):
    # the same special cases on rows long enough for the one-workgroup-per-row kernel, whose grid
    # under a mask holds the compacted selected rows first and the zero-fill of the others after them
    g = seeded(300 + V)
    rows = 7
    s = (torch.randn(1, rows, V, generator=g) * 2).to(dtype)
    t = (torch.randn(1, rows, V, generator=g) * 2).to(dtype)
    sd, td = s.to(device), t.to(device)
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    full = torch.ones(1, rows, dtype=torch.bool)
    a = ta.distil_ce_loss(sd, td, full.to(device), 2.0).item()
    b = ta.kd_soft_target_loss(sd.view(-1, V), td.view(-1, V), 2.0).item()
    assert rel_err(a, b) < 1e-6
    for pick in ([3], [0, 6], [1, 2, 4, 5]):
        m = torch.zeros(1, rows, dtype=torch.bool)
        m[0, pick] = True
        x = sd.clone().requires_grad_()
        l = ta.distil_ce_loss(x, td, m.to(device), 2.0)
        l.backward()
        ref_s = s.double().requires_grad_()
        want = ts_oracle.distil_ce(ref_s, t.double(), m, 2.0)
        want.backward()
        assert rel_err(l.item(), want.item()) < tol
        gw = ref_s.grad
        err = (x.grad.cpu().double() - gw).abs()
        assert (err <= tol * gw.abs().max() + gw.abs() * 2.0 ** -8).all()
        assert (x.grad[0, [i for i in range(rows) if i not in pick]] == 0).all()
    none = torch.zeros(1, rows, dtype=torch.bool)
    x = sd.clone().requires_grad_()
    l = ta.distil_ce_loss(x, td, none.to(device), 2.0)
    l.backward()
    assert torch.isnan(l).item()
    assert (x.grad == 0).all()


def test_byol_fp32(device):
    g = seeded(5)
    o1, o2, t1, t2 = [torch.randn(256, 128, generator=g) for _ in range(4)]
    want, (g1, g2) = _oracle_grad(lambda a, b, c, d: ts_oracle.byol_contrastive_loss(a, b, c, d), o1, o2,
                                  others=(t1, t2))
    d1, d2 = o1.to(device).requires_grad_(), o2.to(device).requires_grad_()
    loss = ta.byol_contrastive_loss(d1, d2, t1.to(device), t2.to(device), None, None)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-5
    assert max_rel_to_peak(d1.grad, g1) < 1e-5 and max_rel_to_peak(d2.grad, g2) < 1e-5
    # gradient is orthogonal to the input row (normalize Jacobian)
    assert (d1.grad * d1.detach()).sum(dim=1).abs().max().item() < 1e-7


def test_byol_special_cases(device):
    x = torch.tensor([[3.0, 4.0, 0.0], [0.0, 2.0, 0.0], [1.0, 0.0, 0.0]], device=device)
    y = torch.stack([x[0] * 2.5, -x[1], torch.tensor([0.0, 0.0, 7.0], device=device)])
    from tspipe_amd.losses import regression_loss_mean
    assert abs(regression_loss_mean(x[:1], y[:1]).item() - 0.0) < 1e-6    # parallel
    assert abs(regression_loss_mean(x[1:2], y[1:2]).item() - 4.0) < 1e-6  # opposite
    assert abs(regression_loss_mean(x[2:], y[2:]).item() - 2.0) < 1e-6    # orthogonal
    # odd width, single row, scale invariance
    g = seeded(6)
    a, b = torch.randn(3, 37, generator=g).to(device), torch.randn(3, 37, generator=g).to(device)
    l1 = regression_loss_mean(a, b).item()
    l2 = regression_loss_mean(a * 7.0, b * 0.25).item()
    assert rel_err(l2, l1) < 1e-5
    want = ts_oracle.byol_regression_loss(a.cpu().double(), b.cpu().double()).mean().item()
    assert rel_err(l1, want) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_byol_and_cosine_over_row_counts_and_widths(device, dtype):
    # a row is a wavefront's work in both kernels (four rows to a workgroup): widths below, at and above
    # what 64 lanes hold in one and in several 16-byte vectors, odd widths (rows off a 16-byte boundary),
    # row counts that leave a workgroup partly empty
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    for n, c in ((1, 1), (2, 3), (5, 64), (3, 65), (7, 255), (4, 256), (9, 257), (6, 768), (2, 1001), (3, 4099)):
        g = seeded(7000 + n + c)
        o1, o2, t1, t2 = [torch.randn(n, c, generator=g).to(dtype) for _ in range(4)]
        want, (g1, g2) = _oracle_grad(ts_oracle.byol_contrastive_loss, o1, o2, others=(t1, t2))
        d1, d2 = o1.to(device).requires_grad_(), o2.to(device).requires_grad_()
        loss = ta.byol_contrastive_loss(d1, d2, t1.to(device), t2.to(device), None, None)
        loss.backward()
        case = f"byol n={n} c={c}"
        assert rel_err(loss.item(), want) < tol or abs(loss.item() - want) < 1e-6, case
        for got, ref, x in ((d1.grad, g1, o1), (d2.grad, g2, o2)):
            slack = ref.abs() * (2.0 ** -8 if dtype != torch.float32 else 0.0)
            # the gradient is a difference of terms of size 2 / (n |x|) per row; at width 1 all of it cancels
            terms = 2.0 / (n * x.double().norm(dim=1, keepdim=True))
            assert ((got.cpu().double() - ref).abs() <= tol * ref.abs().max().item() + slack + tol * 0.1 * terms).all(), case
        # cosine embedding loss with target +1 on the same rows, every other row masked out
        keep = torch.arange(n) % 2 == 0

        def ref_cos(a, b):
            return 1.5 * torch.nn.CosineEmbeddingLoss()(a[keep], b[keep], a.new_ones(int(keep.sum())))
        want, (gx,) = _oracle_grad(ref_cos, o1, others=(t1,))
        xd = o1.to(device).requires_grad_()
        loss = ta.cosine_embedding_loss(xd, t1.to(device), keep.to(device), 1.5)
        loss.backward()
        case = f"cosine n={n} c={c}"
        assert rel_err(loss.item(), want) < tol or abs(loss.item() - want) < 1e-6, case
        slack = gx.abs() * (2.0 ** -8 if dtype != torch.float32 else 0.0)
        terms = 1.5 / (int(keep.sum()) * o1.double().norm(dim=1, keepdim=True))
        assert ((xd.grad.cpu().double() - gx).abs() <= tol * gx.abs().max().item() + slack + tol * 0.1 * terms).all(), case
        assert (xd.grad.cpu()[~keep] == 0).all(), case


def _nce_inputs(n, c, seed, dtype):
    g = seeded(seed)
    q = torch.nn.functional.normalize(torch.randn(n, c, generator=g), dim=1).to(dtype)
    k = torch.nn.functional.normalize(torch.randn(n, c, generator=g), dim=1).to(dtype)
    return q, k


@pytest.mark.parametrize("n,c", [(4096, 256), (1000, 256), (384, 128), (130, 64), (1, 64), (33, 256)])
def test_infonce_bf16(device, n, c):
    q, k = _nce_inputs(n, c, 3, torch.bfloat16)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, 0.2), q, others=(k,))
    qd = q.to(device).requires_grad_()
    loss = ta.infonce_loss(qd, k.to(device), 0.2)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-3 or abs(loss.item() - want) < 1e-6
    peak = gw.abs().max().item()
    err = (qd.grad.cpu().double() - gw).abs()
    assert (err <= 1e-3 * peak + gw.abs() * 2.0 ** -8).all() or peak < 1e-9


@pytest.mark.parametrize("dtype,n,tol", [(torch.bfloat16, 4096, 1e-3), (torch.bfloat16, 1000, 1e-3),
                                         (torch.float32, 640, 1e-4)])
@pytest.mark.parametrize("target", [32, 64, 100])
def test_infonce_workgroup_target_changes_the_schedule_not_the_result(device, dtype, n, tol, target):
    # fewer workgroups = fewer key splits (one at 32): same oracle, same bars
    q, k = _nce_inputs(n, 256, 5, dtype)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, 0.2), q, others=(k,))
    assert ta.set_infonce_workgroup_target(target) == 256
    try:
        qd = q.to(device).requires_grad_()
        loss = ta.infonce_loss(qd, k.to(device), 0.2)
        loss.backward()
        torch.cuda.synchronize()
    finally:
        assert ta.set_infonce_workgroup_target(0) == target
    assert rel_err(loss.item(), want) < (1e-3 if dtype == torch.bfloat16 else 1e-5)
    peak = gw.abs().max().item()
    err = (qd.grad.cpu().double() - gw).abs()
    slack = 2.0 ** -8 if dtype == torch.bfloat16 else 0.0
    assert (err <= tol * peak + gw.abs() * slack).all()


def test_infonce_more_keys_than_an_l2_holds(device):
    # above 8192 rows the launcher makes the key split the fastest grid index; 8330 is not a
    # multiple of the 128-row q tile or the 64-key stage, so padded rows and keys are in play
    n, c = 8330, 256
    q, k = _nce_inputs(n, c, 17, torch.bfloat16)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, 0.2), q, others=(k,))
    qd = q.to(device).requires_grad_()
    loss = ta.infonce_loss(qd, k.to(device), 0.2)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-3
    peak = gw.abs().max().item()
    err = (qd.grad.cpu().double() - gw).abs()
    assert (err <= 1e-3 * peak + gw.abs() * 2.0 ** -8).all()
    # the gradient is orthogonal to its row (normalize Jacobian), a size-independent identity
    dots = (qd.grad.float() * qd.detach().float()).sum(dim=1).abs().max().item()
    assert dots < 2e-2 * peak


def test_infonce_unnormalised_inputs_and_pair(device):
    g = seeded(31)
    o1, o2, t1, t2 = [(torch.randn(512, 256, generator=g) * (0.5 + i)).to(torch.bfloat16) for i in range(4)]
    want, (g1, g2) = _oracle_grad(lambda a, b, c, d: ts_oracle.moco_contrastive_loss(a, b, c, d, 0.2), o1, o2,
                                  others=(t1, t2))
    d1, d2 = o1.to(device).requires_grad_(), o2.to(device).requires_grad_()
    from argparse import Namespace
    loss = ta.moco_contrastive_loss(d1, d2, t1.to(device), t2.to(device), None, Namespace(moco_t=0.2))
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-3
    for got, ref in ((d1.grad, g1), (d2.grad, g2)):
        peak = ref.abs().max().item()
        assert ((got.cpu().double() - ref).abs() <= 1e-3 * peak + ref.abs() * 2.0 ** -8).all()
    # rows of dq are orthogonal to q (normalize Jacobian), up to bf16 storage of dq
    dots = (d1.grad.float() * d1.detach().float()).sum(dim=1).abs().max().item()
    assert dots < 2e-2 * d1.grad.float().abs().max().item() * d1.detach().float().norm(dim=1).max().item()


@pytest.mark.parametrize("n,c", [(512, 256), (130, 64)])
def test_infonce_fp16_inputs(device, n, c):
    # fp16 embeddings (autocast): q and the normalised k are rounded to bf16 for the
    # contraction, as for fp32 inputs, so the tolerance is the bf16 one; dq is stored in fp16
    q, k = _nce_inputs(n, c, 17, torch.float16)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, 0.2), q, others=(k,))
    qd = q.to(device).requires_grad_()
    loss = ta.infonce_loss(qd, k.to(device), 0.2)
    loss.backward()
    assert qd.grad.dtype == torch.float16
    assert rel_err(loss.item(), want) < 2e-3
    assert max_rel_to_peak(qd.grad, gw) < 1e-2


def test_infonce_other_widths_and_argument_errors(device):
    # widths between the kernels' 64 / 128 / 256 are zero-padded (norms and products unchanged)
    for n, c in ((100, 96), (65, 200), (40, 24)):
        q, k = _nce_inputs(n, c, 50 + c, torch.bfloat16)
        want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, 0.2), q, others=(k,))
        qd = q.to(device).requires_grad_()
        loss = ta.infonce_loss(qd, k.to(device), 0.2)
        loss.backward()
        assert qd.grad.shape == (n, c)
        assert rel_err(loss.item(), want) < 1e-3
        err = (qd.grad.cpu().double() - gw).abs()
        assert (err <= 1e-3 * gw.abs().max() + gw.abs() * 2.0 ** -8).all()
    q, k = _nce_inputs(8, 640, 1, torch.bfloat16)
    with pytest.raises(ValueError, match="512 features"):
        ta.infonce_loss(q.to(device), k.to(device), 0.2)
    q, k = _nce_inputs(8, 64, 1, torch.bfloat16)
    with pytest.raises(ValueError, match="temperature"):
        ta.infonce_loss(q.to(device), k.to(device), 0.0)


@pytest.mark.parametrize("dtype,n,c,tau", [
    (torch.bfloat16, 300, 512, 0.2), (torch.bfloat16, 200, 320, 0.2),   # wider than the bf16 kernels
    (torch.bfloat16, 512, 256, 0.01), (torch.float16, 130, 64, 0.02),   # colder than their fixed reference point allows
    (torch.float32, 260, 384, 0.02), (torch.float32, 77, 27, 0.2)])     # both, and a width that is no multiple of 4
def test_infonce_any_width_and_temperature(device, dtype, n, c, tau):
    # what the bf16-MFMA kernels do not take goes to the fp32-MFMA kernels: any --moco-dim up to 512,
    # any --moco-t (benchmarks/moco-v3/main.py:98,107); running maximum, products and sums in fp32
    q, k = _nce_inputs(n, c, 400 + c, dtype)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, tau), q, others=(k,))
    qd = q.to(device).requires_grad_()
    loss = ta.infonce_loss(qd, k.to(device), tau)
    loss.backward()
    assert qd.grad.shape == (n, c) and qd.grad.dtype == dtype
    assert rel_err(loss.item(), want) < 2e-5
    peak = gw.abs().max().item()
    store = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]  # rounding of the stored dq
    err = (qd.grad.cpu().double() - gw).abs()
    # fp16 gradients below the type's subnormal spacing flush: an absolute floor of 2^-24
    assert (err <= 1e-4 * peak + gw.abs() * store + (2.0 ** -24 if dtype == torch.float16 else 0.0)).all()


def test_infonce_fp32_path_over_widths_and_row_counts(device):
    # the fp32-MFMA kernels pad the width to the matrix instruction's step and run widths above 256 as two
    # feature groups; rows come in tiles of 32 per wavefront, 128 per workgroup: every edge of both
    for n, c in ((1, 1), (2, 2), (31, 3), (33, 5), (32, 31), (129, 33), (127, 63), (5, 65), (64, 127), (65, 129),
                 (40, 255), (128, 257), (130, 320), (3, 511), (97, 512)):
        q, k = _nce_inputs(n, c, 5000 + n + c, torch.float32)
        want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, 0.2), q, others=(k,))
        qd = q.to(device).requires_grad_()
        loss = ta.infonce_loss(qd, k.to(device), 0.2)
        loss.backward()
        case = f"n={n} c={c}"
        assert rel_err(loss.item(), want) < 2e-5 or abs(loss.item() - want) < 1e-6, case
        # at width 1 the whole gradient is the projected-out component: bounded by its terms, 2 tau / (n tau |q|)
        terms = 2.0 / (n * q.double().norm(dim=1, keepdim=True))
        assert ((qd.grad.cpu().double() - gw).abs() <= 1e-4 * gw.abs().max().item() + 1e-6 * terms).all(), case


@pytest.mark.parametrize("n,c,tau", [(1000, 256, 0.2), (4096, 256, 0.2), (300, 128, 0.07), (130, 64, 0.5), (1, 64, 0.2)])
def test_infonce_fp32_inputs_in_fp32_arithmetic(device, n, c, tau):
    # the reference's TSPipe MoCo run is fp32 end to end (benchmarks/moco-v3/main.py:151-160, no autocast):
    # fp32 embeddings are contracted on the fp32 matrix instruction, nothing is rounded to bf16
    q, k = _nce_inputs(n, c, 40 + n, torch.float32)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, tau), q, others=(k,))
    qd = q.to(device).requires_grad_()
    loss = ta.infonce_loss(qd, k.to(device), tau)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-5 or abs(loss.item() - want) < 1e-6
    assert max_rel_to_peak(qd.grad, gw) < 1e-4 or gw.abs().max() < 1e-9
    # the gradient is orthogonal to its row (normalize Jacobian)
    if n > 1:
        dots = (qd.grad * qd.detach()).sum(dim=1).abs().max().item()
        assert dots < 1e-5 * gw.abs().max().item()


def test_infonce_fp32_inputs_and_identities(device):
    q, k = _nce_inputs(256, 128, 9, torch.float32)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, 0.5), q, others=(k,))
    qd = q.to(device).requires_grad_()
    loss = ta.infonce_loss(qd, k.to(device), 0.5)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-5
    assert max_rel_to_peak(qd.grad, gw) < 1e-4
    # N = 1: a single logit, loss 0
    q1, k1 = _nce_inputs(1, 64, 10, torch.bfloat16)
    assert abs(ta.infonce_loss(q1.to(device), k1.to(device), 0.2).item()) < 1e-6
    # scale invariance in q and k
    qb, kb = _nce_inputs(200, 64, 12, torch.bfloat16)
    l1 = ta.infonce_loss(qb.to(device), kb.to(device), 0.2).item()
    l2 = ta.infonce_loss((qb * 4).to(device), (kb * 0.5).to(device), 0.2).item()
    assert rel_err(l2, l1) < 1e-4


# ---- KD + hard-label CE in one pass, cosine loss, the full loss_fn plug-ins ----

@pytest.mark.parametrize("rows,V,dtype", [(256, 100, torch.float32), (37, 1000, torch.float32), (9, 5000, torch.float32),
                                          (64, 30522, torch.bfloat16)])
def test_soft_target_tspipe_loss(device, rows, V, dtype):
    from argparse import Namespace
    g = seeded(200 + V)
    s = (torch.randn(rows, V, generator=g) * 3).to(dtype)
    t = (torch.randn(rows, V, generator=g) * 3).to(dtype)
    y = torch.randint(0, V, (rows,), generator=g)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.soft_target_tspipe_loss(a, b, y, 4.0, 0.7), s, others=(t,))
    sd = s.to(device).requires_grad_()
    args = Namespace(kd_mode="st", T=4.0, lambda_kd=0.7)
    loss = ta.soft_target_tspipe_loss(sd, t.to(device), y.to(device), None, args, 0)
    loss.backward()
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    assert rel_err(loss.item(), want) < tol
    peak = gw.abs().max().item()
    slack = gw.abs() * (2.0 ** -8 if dtype != torch.float32 else 0.0)
    assert ((sd.grad.cpu().double() - gw).abs() <= tol * peak + slack).all()


def test_kd_ce_row_sets_and_ignore_index(device):
    g = seeded(210)
    rows, V = 40, 257
    s = torch.randn(rows, V, generator=g) * 2
    t = torch.randn(rows, V, generator=g) * 2
    mask = torch.rand(rows, generator=g) < 0.4
    y = torch.randint(0, V, (rows,), generator=g)
    y[torch.rand(rows, generator=g) < 0.5] = -100
    assert (mask & (y == -100)).any() and (~mask & (y != -100)).any() and (~mask & (y == -100)).any()

    def ref(a, b):
        kd = ts_oracle.distil_ce(a.view(1, rows, V), b.view(1, rows, V), mask.view(1, rows), 2.0, 0.5)
        ce = torch.nn.CrossEntropyLoss(ignore_index=-100)(a, y)
        return kd + 2.0 * ce
    want, (gw,) = _oracle_grad(ref, s, others=(t,))
    sd = s.to(device).requires_grad_()
    loss = ta.kd_ce_loss(sd, t.to(device), y.to(device), 2.0, kd_weight=0.5, ce_weight=2.0, row_mask=mask.to(device))
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-5
    assert max_rel_to_peak(sd.grad, gw) < 1e-5
    idle = ~mask & (y == -100)
    assert (sd.grad.cpu()[idle] == 0).all()
    # no valid label at all: the CE mean is 0/0 = NaN, as torch gives
    none = torch.full((rows,), -100, dtype=torch.long)
    l = ta.kd_ce_loss(s.to(device), t.to(device), none.to(device), 2.0, row_mask=mask.to(device))
    assert torch.isnan(l).item() and torch.isnan(torch.nn.CrossEntropyLoss(ignore_index=-100)(s, none)).item()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kd_ce_mse_at_every_row_width_boundary(device, dtype):
    # The launcher picks a kernel by the number of 16-byte vectors a row can span: 16-, 32- and 64-lane
    # groups, a 256-thread workgroup, 512 and 1024 threads with the row in registers, two passes beyond.
    # Every boundary from both sides, with all three terms at once (KD under a mask, cross entropy with
    # ignored labels, squared error), rows that start off a 16-byte boundary because the width is odd,
    # and once more with the student one element off the teacher's alignment.
    vec = 16 // torch.empty((), dtype=dtype).element_size()
    widths = []
    for vecs in (32, 64, 256, 1024, 4096, 8192):   # largest ceil(V / vec) + 1 each kernel takes
        widths += [(vecs - 1) * vec, (vecs - 1) * vec + 1]
    widths += [8191, 8192, 8193]                   # the squared-error term's own threshold (elements)
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    rows = 5
    for V in widths:
        for shift in (0, 1):
            g = seeded(9000 + V + shift)
            s = (torch.randn(rows, V, generator=g) * 2).to(dtype)
            t = (torch.randn(rows, V, generator=g) * 2).to(dtype)
            mask = torch.tensor([True, False, True, True, False])
            y = torch.tensor([V - 1, 0, -100, V // 2, -100])

            def ref(a, b):
                kd = ts_oracle.distil_ce(a.view(1, rows, V), b.view(1, rows, V), mask.view(1, rows), 2.0, 0.5)
                ce = torch.nn.CrossEntropyLoss(ignore_index=-100)(a, y)
                d = (a[mask] - b[mask])
                return kd + 2.0 * ce + 0.05 * (d * d).sum() / int(mask.sum())
            want, (gw,) = _oracle_grad(ref, s, others=(t,))
            buf = torch.zeros(rows * V + 8, dtype=dtype, device=device)
            sd = buf[shift:shift + rows * V].view(rows, V)
            sd.copy_(s)
            sd = sd.detach().requires_grad_()
            loss = ta.kd_ce_loss(sd, t.to(device), y.to(device), 2.0, kd_weight=0.5, ce_weight=2.0,
                                 row_mask=mask.to(device), mse_weight=0.05)
            loss.backward()
            case = f"V={V} shift={shift}"
            assert rel_err(loss.item(), want) < tol, case
            peak = gw.abs().max().item()
            # 16-bit gradients: the squared-error term is added to a KD + CE gradient already stored
            slack = gw.abs() * (2.0 ** -7 if dtype != torch.float32 else 0.0)
            assert ((sd.grad.cpu().double() - gw).abs() <= tol * peak + slack).all(), case
            assert (sd.grad.cpu()[4] == 0).all(), case   # neither masked in nor labelled


@pytest.mark.parametrize("rows", [77, 1027, 2048, 2049, 8195])  # 2048: the last batch size whose workgroups count for themselves
def test_kd_ce_counts_from_a_mask_that_starts_off_an_8_byte_boundary(device, rows):
    # short rows under a mask and with labels take a counting launch that reads the mask eight rows at a
    # time when it can; a mask that is a view three bytes into a buffer cannot, and must count the same
    g = seeded(930 + rows)
    V = 50
    s = torch.randn(rows, V, generator=g).to(device)
    t = torch.randn(rows, V, generator=g).to(device)
    mask = (torch.rand(rows, generator=g) < 0.4).to(device)
    y = torch.randint(0, V, (rows,), generator=g)
    y[torch.rand(rows, generator=g) < 0.5] = -100
    y = y.to(device)
    big = torch.zeros(rows + 16, dtype=torch.bool, device=device)
    off = big[3:3 + rows]
    off.copy_(mask)
    assert off.data_ptr() % 8 == 3 and mask.data_ptr() % 8 == 0
    a = s.clone().requires_grad_()
    la = ta.kd_ce_loss(a, t, y, 2.0, kd_weight=0.5, ce_weight=2.0, row_mask=mask)
    la.backward()
    b = s.clone().requires_grad_()
    lb = ta.kd_ce_loss(b, t, y, 2.0, kd_weight=0.5, ce_weight=2.0, row_mask=off)
    lb.backward()
    assert torch.equal(la, lb) and torch.equal(a.grad, b.grad)
    # and against the closed form of the two means
    sm, tm = s.cpu().double(), t.cpu().double()
    m, yy = mask.cpu(), y.cpu()
    kd = torch.nn.functional.kl_div(torch.log_softmax(sm[m] / 2.0, -1), torch.softmax(tm[m] / 2.0, -1),
                                    reduction="batchmean") * 4.0
    ce = torch.nn.functional.cross_entropy(sm, yy, ignore_index=-100)
    assert rel_err(la.item(), (0.5 * kd + 2.0 * ce).item()) < 1e-5


def test_cosine_embedding_loss(device):
    g = seeded(220)
    x = torch.randn(3, 7, 48, generator=g)
    y = torch.randn(3, 7, 48, generator=g)
    att = torch.rand(3, 7, generator=g) < 0.6

    def ref(a, b):
        m = att.unsqueeze(-1).expand_as(a)
        a2, b2 = torch.masked_select(a, m).view(-1, 48), torch.masked_select(b, m).view(-1, 48)
        return 1.5 * torch.nn.CosineEmbeddingLoss()(a2, b2, a2.new_ones(a2.size(0)))
    want, (gw,) = _oracle_grad(ref, x, others=(y,))
    xd = x.to(device).requires_grad_()
    loss = ta.cosine_embedding_loss(xd, y.to(device), att.to(device), 1.5)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-5
    assert max_rel_to_peak(xd.grad, gw) < 1e-5
    assert (xd.grad.cpu()[~att] == 0).all()
    full = ta.cosine_embedding_loss(x.to(device), y.to(device)).item()
    assert rel_err(full, torch.nn.CosineEmbeddingLoss()(x.view(-1, 48).double(), y.view(-1, 48).double(),
                                                      torch.ones(21, dtype=torch.float64)).item()) < 1e-5


@pytest.mark.parametrize("restrict", [True, False])
def test_distil_loss_fn_plugin(device, restrict):
    from argparse import Namespace
    g = seeded(230)
    bs, seq, V, H = 4, 16, 30522, 64
    s = (torch.randn(bs, seq, V, generator=g) * 2).to(torch.bfloat16)
    t = (torch.randn(bs, seq, V, generator=g) * 2).to(torch.bfloat16)
    sh = torch.randn(bs, seq, H, generator=g).to(torch.bfloat16)
    th = torch.randn(bs, seq, H, generator=g).to(torch.bfloat16)
    lm = torch.full((bs, seq), -100, dtype=torch.long)
    pick = torch.rand(bs, seq, generator=g) < 0.15
    lm[pick] = torch.randint(0, V, (int(pick.sum()),), generator=g)
    att = torch.rand(bs, seq, generator=g) < 0.8
    params = Namespace(alpha_ce=0.5, alpha_mlm=2.0, alpha_clm=0.0, alpha_mse=0.0, alpha_cos=1.0, temperature=2.0,
                       restrict_ce_to_mask=restrict)
    want, (gs, gh) = _oracle_grad(
        lambda a, h, b, hb: ts_oracle.distil_loss(a, b, h, hb, lm, att, 0.5, 2.0, 1.0, 2.0, restrict), s, sh,
        others=(t, th))
    sd, shd = s.to(device).requires_grad_(), sh.to(device).requires_grad_()
    loss = ta.distil_loss_fn({"logits": sd, "hidden_states": (shd,)},
                             {"logits": t.to(device), "hidden_states": (th.to(device),)},
                             (lm.to(device), att.to(device)), None, params, 0)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-3
    for got, ref in ((sd.grad, gs), (shd.grad, gh)):
        peak = ref.abs().max().item()
        assert ((got.cpu().double() - ref).abs() <= 1e-3 * peak + ref.abs() * 2.0 ** -8).all()


@pytest.mark.parametrize("mode", ["clm", "mse", "clm+mse"])
def test_distil_loss_fn_clm_and_mse_terms(device, mode):
    from argparse import Namespace
    g = seeded(231)
    bs, seq, V = 3, 12, 5000
    s = (torch.randn(bs, seq, V, generator=g) * 2).to(torch.bfloat16)
    t = (torch.randn(bs, seq, V, generator=g) * 2).to(torch.bfloat16)
    lm = torch.full((bs, seq), -100, dtype=torch.long)
    pick = torch.rand(bs, seq, generator=g) < 0.3
    lm[pick] = torch.randint(0, V, (int(pick.sum()),), generator=g)
    att = torch.rand(bs, seq, generator=g) < 0.8
    a_clm = 1.5 if "clm" in mode else 0.0
    a_mse = 0.05 if "mse" in mode else 0.0
    params = Namespace(alpha_ce=0.5, alpha_mlm=0.0, alpha_clm=a_clm, alpha_mse=a_mse, alpha_cos=0.0, temperature=2.0,
                       restrict_ce_to_mask=False)
    want, (gs,) = _oracle_grad(
        lambda a, b: ts_oracle.distil_loss(a, b, None, None, lm, att, 0.5, 0.0, 0.0, 2.0, False, alpha_clm=a_clm,
                                           alpha_mse=a_mse), s, others=(t,))
    sd = s.to(device).requires_grad_()
    loss = ta.distil_loss_fn({"logits": sd, "hidden_states": None}, {"logits": t.to(device), "hidden_states": None},
                             (lm.to(device), att.to(device)), None, params, 0)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-3
    peak = gs.abs().max().item()
    # the MSE term is added to a gradient already stored in bf16: two roundings
    assert ((sd.grad.cpu().double() - gs).abs() <= 1e-3 * peak + gs.abs() * 2.0 ** -7).all()
    # both hard-label terms at once, as the reference's loss_fn adds them (distiller.py:742-749)
    params.alpha_mlm, params.alpha_clm = 0.7, 1.5
    want, (gs,) = _oracle_grad(
        lambda a, b: ts_oracle.distil_loss(a, b, None, None, lm, att, 0.5, 0.7, 0.0, 2.0, False, alpha_clm=1.5,
                                           alpha_mse=a_mse), s, others=(t,))
    sd = s.to(device).requires_grad_()
    loss = ta.distil_loss_fn({"logits": sd, "hidden_states": None}, {"logits": t.to(device), "hidden_states": None},
                             (lm.to(device), att.to(device)), None, params, 0)
    loss.backward()
    assert rel_err(loss.item(), want) < 1e-3
    peak = gs.abs().max().item()
    assert ((sd.grad.cpu().double() - gs).abs() <= 1e-3 * peak + gs.abs() * 2.0 ** -6).all()


def test_logits_mse_operands_aligned_differently(device):
    # s and t at different offsets from a 16-byte boundary (views into larger buffers): the kernel
    # walks such rows element by element; rows of 2051 elements also exercise a second span, rows of 8200
    # the kernel that gives a row a workgroup of its own
    g = seeded(77)
    for rows, V, dtype, tol in ((9, 2051, torch.float32, 1e-5), (9, 2051, torch.bfloat16, 1e-3),
                                (3, 8200, torch.float32, 1e-5), (3, 8200, torch.bfloat16, 1e-3)):  # a workgroup per row
        s = (torch.randn(rows, V, generator=g) * 3).to(dtype)
        t = (torch.randn(rows, V, generator=g) * 3).to(dtype)
        want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.logits_mse(a, b), s, others=(t,))
        buf_s = torch.zeros(rows * V + 8, dtype=dtype, device=device)
        buf_t = torch.zeros(rows * V + 8, dtype=dtype, device=device)
        sd = buf_s[1:1 + rows * V].view(rows, V)
        td = buf_t[3:3 + rows * V].view(rows, V)
        sd.copy_(s)
        td.copy_(t)
        sd = sd.detach().requires_grad_()
        loss = ta.logits_mse_loss(sd, td)
        loss.backward()
        assert rel_err(loss.item(), want) < tol
        slack = gw.abs() * (2.0 ** -8 if dtype != torch.float32 else 0.0)
        assert ((sd.grad.cpu().double() - gw).abs() <= tol * gw.abs().max().item() + slack).all()


@pytest.mark.parametrize("rows,V,dtype", [(256, 100, torch.float32), (33, 5000, torch.float32),
                                          (40, 30522, torch.bfloat16), (37, 101, torch.float32),
                                          (19, 1001, torch.bfloat16),
                                          # rows of 8192 elements and more take a workgroup each: the threshold itself,
                                          # rows that start at every offset from a 16-byte boundary, more vectors than
                                          # one round of loads holds
                                          (5, 8192, torch.float32), (7, 9001, torch.float32),
                                          (3, 40003, torch.bfloat16), (2, 20000, torch.float16)])
def test_logits_mse_and_kd_mode_logits(device, rows, V, dtype):
    from argparse import Namespace
    g = seeded(240 + V)
    s = (torch.randn(rows, V, generator=g) * 3).to(dtype)
    t = (torch.randn(rows, V, generator=g) * 3).to(dtype)
    y = torch.randint(0, V, (rows,), generator=g)
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    # the criterion alone (kd_losses/logits.py), module form
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.logits_mse(a, b), s, others=(t,))
    sd = s.to(device).requires_grad_()
    loss = ta.Logits()(sd, t.to(device))
    loss.backward()
    assert rel_err(loss.item(), want) < tol
    peak = gw.abs().max().item()
    slack = gw.abs() * (2.0 ** -8 if dtype != torch.float32 else 0.0)
    assert ((sd.grad.cpu().double() - gw).abs() <= tol * peak + slack).all()
    # masked rows, sum over columns / selected rows; zero gradient elsewhere
    mask = torch.rand(rows, generator=g) < 0.5
    sm, tm = s[mask].double(), t[mask].double()
    sd2 = s.to(device).requires_grad_()
    l2 = ta.logits_mse_loss(sd2, t.to(device), mask.to(device), weight=0.5, per_element=False)
    l2.backward()
    assert rel_err(l2.item(), 0.5 * ((sm - tm) ** 2).sum().item() / int(mask.sum())) < tol
    assert (sd2.grad.cpu()[~mask] == 0).all()
    gwant = 0.5 * 2 * (sm - tm) / int(mask.sum())
    assert ((sd2.grad.cpu()[mask].double() - gwant).abs() <= tol * gwant.abs().max() + gwant.abs() * 2.0 ** -8).all()
    # the whole plug-in with kd_mode == 'logits'
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.soft_target_tspipe_loss(a, b, y, 4.0, 0.7, kd_mode="logits"), s,
                               others=(t,))
    sd3 = s.to(device).requires_grad_()
    args = Namespace(kd_mode="logits", T=4.0, lambda_kd=0.7)
    loss = ta.soft_target_tspipe_loss(sd3, t.to(device), y.to(device), None, args, 0)
    loss.backward()
    assert rel_err(loss.item(), want) < tol
    peak = gw.abs().max().item()
    slack = gw.abs() * (2.0 ** -7 if dtype != torch.float32 else 0.0)
    assert ((sd3.grad.cpu().double() - gw).abs() <= tol * peak + slack).all()


@pytest.mark.parametrize("rows,V,dtype,with_ce", [((64, 64, 64, 64), 100, torch.float32, True),
                                                  ((5, 1, 9, 2, 7, 3, 4, 6), 1000, torch.float32, False),
                                                  ((8, 8, 8, 5), 30522, torch.bfloat16, True),
                                                  ((3,), 6000, torch.bfloat16, False)])
def test_kd_pieces_equal_gathered(device, rows, V, dtype, with_ce):
    # micro-batch outputs that are never concatenated: same loss and gradient
    # as the kernel on the gathered tensors, bit for bit (same arithmetic, only
    # the row addresses differ; the shapes here keep every row at the same
    # 16-byte phase in both layouts, so even the summation order is the same),
    # and within the usual bar of the oracle
    g = seeded(250 + V)
    s_p = [(torch.randn(r, V, generator=g) * 2).to(dtype) for r in rows]
    t_p = [(torch.randn(r, V, generator=g) * 2).to(dtype) for r in rows]
    total = sum(rows)
    mask = torch.rand(total, generator=g) < 0.5
    labels = None
    if with_ce:
        labels = torch.randint(0, V, (total,), generator=g)
        labels[torch.rand(total, generator=g) < 0.4] = -100
    sd = [p.to(device).requires_grad_() for p in s_p]
    td = [p.to(device) for p in t_p]
    lab_d = None if labels is None else labels.to(device)
    loss = ta.kd_ce_loss_pieces(sd, td, lab_d, 2.0, kd_weight=0.5, ce_weight=1.5, row_mask=mask.to(device))
    loss.backward()
    s_cat = torch.cat([p.to(device) for p in s_p]).requires_grad_()
    ref = ta.kd_ce_loss(s_cat, torch.cat(td), lab_d, 2.0, kd_weight=0.5, ce_weight=1.5, row_mask=mask.to(device))
    ref.backward()
    assert loss.item() == ref.item()
    assert torch.equal(torch.cat([p.grad for p in sd]), s_cat.grad)

    def oracle(a, b):
        out = ts_oracle.distil_ce(a, b, mask, 2.0, 0.5)
        if labels is not None:
            out = out + 1.5 * torch.nn.CrossEntropyLoss(ignore_index=-100)(a, labels)
        return out
    want, (gw,) = _oracle_grad(oracle, torch.cat(s_p), others=(torch.cat(t_p),))
    tol = 1e-5 if dtype == torch.float32 else 1e-3
    assert rel_err(loss.item(), want) < tol
    got = torch.cat([p.grad for p in sd]).cpu().double()
    slack = gw.abs() * (2.0 ** -8 if dtype != torch.float32 else 0.0)
    assert ((got - gw).abs() <= tol * gw.abs().max().item() + slack).all()


@pytest.mark.parametrize("a_mse,restrict", [(0.0, True), (0.25, True), (0.25, False)])
def test_distil_loss_fn_pieces_matches_gathered_plugin(device, a_mse, restrict):
    # every term reads the micro-batch outputs where they lie (KD, CE and squared error on the logits,
    # cosine on the hidden states): bit-equal to the same plug-in on the concatenated tensors
    from argparse import Namespace
    g = seeded(260)
    chunks, bs, seq, V, H = 4, 2, 16, 30522, 32
    s = [(torch.randn(bs, seq, V, generator=g) * 2).to(torch.bfloat16).to(device).requires_grad_() for _ in range(chunks)]
    t = [(torch.randn(bs, seq, V, generator=g) * 2).to(torch.bfloat16).to(device) for _ in range(chunks)]
    sh = [torch.randn(bs, seq, H, generator=g).to(torch.bfloat16).to(device).requires_grad_() for _ in range(chunks)]
    th = [torch.randn(bs, seq, H, generator=g).to(torch.bfloat16).to(device) for _ in range(chunks)]
    lm = torch.full((chunks * bs, seq), -100, dtype=torch.long)
    pick = torch.rand(chunks * bs, seq, generator=g) < 0.15
    lm[pick] = torch.randint(0, V, (int(pick.sum()),), generator=g)
    att = torch.rand(chunks * bs, seq, generator=g) < 0.8
    params = Namespace(alpha_ce=0.5, alpha_mlm=2.0, alpha_clm=0.0, alpha_mse=a_mse, alpha_cos=1.0, temperature=2.0,
                       restrict_ce_to_mask=restrict)
    labels = (lm.to(device), att.to(device))
    loss = ta.distil_loss_fn_pieces([{"logits": a, "hidden_states": (b,)} for a, b in zip(s, sh)],
                                    [{"logits": a, "hidden_states": (b,)} for a, b in zip(t, th)], labels, None, params, 0)
    loss.backward()
    s_cat = torch.cat([p.detach() for p in s]).requires_grad_()
    sh_cat = torch.cat([p.detach() for p in sh]).requires_grad_()
    ref = ta.distil_loss_fn({"logits": s_cat, "hidden_states": (sh_cat,)},
                            {"logits": torch.cat(t), "hidden_states": (torch.cat(th),)}, labels, None, params, 0)
    ref.backward()
    assert loss.item() == ref.item()
    assert torch.equal(torch.cat([p.grad for p in s]), s_cat.grad)
    assert torch.equal(torch.cat([p.grad for p in sh]), sh_cat.grad)
    # and the gathered plug-in against the oracle on a slice the fp64 evaluation can afford is
    # test_distil_loss_fn_plugin's job; here the cosine and squared-error pieces alone, against it
    x = [p.detach().float().cpu() for p in sh]
    y = [p.float().cpu() for p in th]
    xc = torch.cat(x).double().requires_grad_()
    keep = att.reshape(-1)
    cosv = torch.nn.functional.cosine_similarity(xc.reshape(-1, H)[keep], torch.cat(y).double().reshape(-1, H)[keep], dim=1)
    want = (1.0 - cosv).mean()
    want.backward()
    xs = [p.detach().clone().requires_grad_() for p in sh]
    got = ta.cosine_embedding_loss_pieces(xs, th, att.to(device))
    got.backward()
    assert rel_err(got.item(), want.item()) < 1e-3
    gp = torch.cat([p.grad for p in xs]).double().cpu()
    assert ((gp - xc.grad).abs() <= 1e-3 * xc.grad.abs().max() + xc.grad.abs() * 2.0 ** -8).all()


def test_kd_pieces_argument_errors(device):
    s = [torch.randn(4, 10, device=device) for _ in range(9)]
    with pytest.raises(Exception):
        ta.kd_ce_loss_pieces(s, s, None, 2.0)  # more than 8 pieces
    with pytest.raises(ValueError):
        ta.kd_ce_loss_pieces(s[:2], s[:3], None, 2.0)
    with pytest.raises(ValueError):
        ta.kd_ce_loss_pieces(s[:2], s[:2], None, 2.0, row_mask=torch.ones(7, dtype=torch.bool, device=device))


def test_kd_masked_cfg3_full_size_properties(device):
    # [32, 128, 30522] bf16, 15 % token mask, gathered from 4 micro-batches: too large for the
    # fp64 oracle, so checked through properties that do not depend on the size
    g = seeded(2)
    pieces_s = [(torch.randn(8, 128, 30522, generator=g) * 2).to(torch.bfloat16).to(device) for _ in range(4)]
    pieces_t = [(torch.randn(8, 128, 30522, generator=g) * 2).to(torch.bfloat16).to(device) for _ in range(4)]
    mask = (torch.rand(32, 128, generator=g) < 0.15).to(device)
    s = ta.gather([ta.Batch(p) for p in pieces_s]).requires_grad_()
    t = ta.gather([ta.Batch(p) for p in pieces_t])
    loss = ta.distil_ce_loss(s, t, mask, 2.0)
    loss.backward()
    n_sel = int(mask.sum())
    assert 400 < n_sel < 900
    # (1) same rows through the unmasked narrow-free path: compact them with torch indexing first
    s_sel = s.detach()[mask].clone().requires_grad_()
    t_sel = t[mask].clone()
    loss2 = ta.kd_soft_target_loss(s_sel, t_sel, 2.0)
    loss2.backward()
    assert rel_err(loss.item(), loss2.item()) < 1e-5
    # same arithmetic up to summation order (the compacted rows are aligned differently): one bf16 ulp
    assert torch.allclose(s.grad[mask].float(), s_sel.grad.float(), rtol=2.0 ** -7, atol=1e-12)
    # (2) nothing outside the mask, (3) gradient rows sum to ~0, (4) loss > 0
    assert (s.grad[~mask] == 0).all()
    sums = s.grad[mask].float().sum(dim=1).abs().max().item()
    assert sums < 5e-3 * s.grad[mask].float().abs().sum(dim=1).max().item()
    assert loss.item() > 0
    # (5) a 64-row sample against the fp64 oracle
    rows = mask.reshape(-1).nonzero().squeeze(1)[:64].cpu()
    ss = s.detach().reshape(-1, 30522)[rows.to(device)].cpu().double().requires_grad_()
    tt = t.reshape(-1, 30522)[rows.to(device)].cpu().double()
    (ts_oracle.kd_soft_target(ss, tt, 2.0) * 64 / n_sel).backward()
    got = s.grad.reshape(-1, 30522)[rows.to(device)].cpu().double()
    peak = ss.grad.abs().max().item()
    assert ((got - ss.grad).abs() <= 1e-3 * peak + ss.grad.abs() * 2.0 ** -8).all()


@pytest.mark.parametrize("dtype,tau,noise,tol", [
    # (k = q + noise: the teacher nearly agrees with the student, the regime of a trained model)
    (torch.bfloat16, 0.2, 0.01, 6e-3), (torch.bfloat16, 0.2, 1.0, 4e-3),
    (torch.float32, 0.2, 0.01, 1e-4), (torch.float32, 0.2, 1.0, 1e-4),
    (torch.bfloat16, 0.07, 0.1, 1.5e-2), (torch.float32, 0.07, 0.1, 1e-3)])
def test_infonce_nearly_aligned_pairs(device, dtype, tau, noise, tol):
    # With k_i close to q_i the gradient is what is left after two cancellations: the positive key
    # against its own soft-max weight, and the component along q that the normalisation projects out.
    # The kernel keeps the positive key in fp32 and takes the projection from the gradient itself, so
    # the error stays a few bf16 roundings (2^-9) of the NEGATIVE keys' weighted sum.  Bounds measured
    # on MI355X (error over the gradient's peak): 2.3e-3 .. 3.9e-3 at tau = 0.2, 1.1e-2 at tau = 0.07,
    # where the peak itself is 1e-7; the previous formulation (positive key rounded with the others,
    # projection from separately accumulated sums) gave 2.7e-2 and 1.8e+2 there.  fp32 embeddings run in
    # fp32 arithmetic throughout and meet the bar of the other loss tests.
    n, c = 512, 256
    g = seeded(77)
    q = torch.nn.functional.normalize(torch.randn(n, c, generator=g), dim=1)
    k = torch.nn.functional.normalize(q + noise * torch.randn(n, c, generator=g) / 16, dim=1)
    q, k = q.to(dtype), k.to(dtype)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, tau), q, others=(k,))
    qd = q.to(device).requires_grad_()
    loss = ta.infonce_loss(qd, k.to(device), tau)
    loss.backward()
    assert abs(loss.item() - want) < 1e-3 * abs(want) + 1e-6
    assert max_rel_to_peak(qd.grad, gw) < tol


@pytest.mark.parametrize("dtype,tau,noise", [(torch.bfloat16, 0.2, 0.01), (torch.bfloat16, 0.2, 1.0),
                                             (torch.bfloat16, 0.07, 0.1), (torch.float16, 0.2, 0.01)])
def test_infonce_fp32_arithmetic_switch_on_16_bit_pairs(device, dtype, tau, noise):
    # the same nearly aligned pairs with the accuracy switch on: 16-bit embeddings on the fp32-MFMA
    # kernels.  What is left is the storage rounding of dq itself (2^-9 of each element for bf16)
    # on top of the fp32 path's 1e-4 of the peak (1e-3 at tau = 0.07), instead of 4e-3 .. 1.5e-2 of
    # the peak on the bf16-MFMA kernels.
    n, c = 512, 256
    g = seeded(77)
    q = torch.nn.functional.normalize(torch.randn(n, c, generator=g), dim=1)
    k = torch.nn.functional.normalize(q + noise * torch.randn(n, c, generator=g) / 16, dim=1)
    q, k = q.to(dtype), k.to(dtype)
    want, (gw,) = _oracle_grad(lambda a, b: ts_oracle.infonce(a, b, tau), q, others=(k,))
    assert ta.set_infonce_fp32_arithmetic(True) is False
    try:
        qd = q.to(device).requires_grad_()
        loss = ta.infonce_loss(qd, k.to(device), tau)
        loss.backward()
        # and the un-gathered form takes the same route
        qp = [p.contiguous().requires_grad_() for p in q.to(device).split([200, 312])]
        kp = [p.contiguous() for p in k.to(device).split([200, 312])]
        from argparse import Namespace
        lp = ta.moco_contrastive_loss_pieces(qp, qp, kp, kp, None, Namespace(moco_t=tau))
        lp.backward()
    finally:
        assert ta.set_infonce_fp32_arithmetic(False) is True
    assert abs(loss.item() - want) < 1e-5 * abs(want) + 1e-7
    assert abs(lp.item() - 2 * want) < 1e-5 * abs(2 * want) + 1e-7  # both directions were the same pair
    peak = gw.abs().max().item()
    slack = 1e-4 if tau >= 0.2 else 1e-3
    # (an fp16 gradient this small is stored in subnormals: their spacing, 2^-24, joins the bound)
    floor = 2.0 ** -24 if dtype == torch.float16 else 0.0
    assert ((qd.grad.cpu().double() - gw).abs() <= slack * peak + gw.abs() * 2.0 ** -8 + floor).all()
    # the switch is off again: the same call is back on the bf16-MFMA kernels (a different rounding)
    qd2 = q.to(device).requires_grad_()
    ta.infonce_loss(qd2, k.to(device), tau).backward()
    assert not torch.equal(qd2.grad, qd.grad)


@pytest.mark.parametrize("dtype,c,rows", [(torch.bfloat16, 256, [96, 32, 100, 28]), (torch.float32, 128, [40, 40, 17]),
                                         (torch.bfloat16, 64, [64])])
def test_moco_loss_on_pieces_equals_the_gathered_loss(device, dtype, c, rows):
    from argparse import Namespace
    n = sum(rows)
    g = seeded(500 + c)
    full = [torch.randn(n, c, generator=g).to(dtype) for _ in range(4)]  # o1, o2, t1, t2
    extra = Namespace(moco_t=0.2)
    # the oracle on the concatenated tensors
    want, grads = _oracle_grad(lambda a, b, t1, t2: ts_oracle.moco_contrastive_loss(a, b, t1, t2, 0.2),
                               full[0], full[1], others=(full[2], full[3]))
    # the gathered kernel
    o1, o2 = full[0].to(device).requires_grad_(), full[1].to(device).requires_grad_()
    whole = ta.moco_contrastive_loss(o1, o2, full[2].to(device), full[3].to(device), None, extra)
    whole.backward()
    # the same from the pieces, never concatenated
    split = lambda t: [p.contiguous().to(device) for p in t.split(rows)]  # noqa: E731
    p1, p2 = [p.requires_grad_() for p in split(full[0])], [p.requires_grad_() for p in split(full[1])]
    loss = ta.moco_contrastive_loss_pieces(p1, p2, split(full[2]), split(full[3]), None, extra)
    loss.backward()
    assert torch.equal(loss, whole)
    assert torch.equal(torch.cat([p.grad for p in p1]), o1.grad)
    assert torch.equal(torch.cat([p.grad for p in p2]), o2.grad)
    tol = 1e-3 if dtype == torch.bfloat16 else 1e-4  # fp32 inputs run in fp32 arithmetic
    assert rel_err(loss.item(), want) < tol
    for got, ref in ((o1.grad, grads[0]), (o2.grad, grads[1])):
        peak = ref.abs().max().item()
        assert ((got.cpu().double() - ref).abs() <= tol * peak + ref.abs() * (2.0 ** -8 if dtype == torch.bfloat16 else 0)).all()


def test_byol_loss_on_pieces_equals_the_gathered_loss(device):
    rows = [100, 28, 64, 64]
    n, c = sum(rows), 128
    g = seeded(611)
    full = [torch.randn(n, c, generator=g) for _ in range(4)]  # o1, o2, t1, t2
    want, grads = _oracle_grad(ts_oracle.byol_contrastive_loss, full[0], full[1], others=(full[2], full[3]))
    o1, o2 = full[0].to(device).requires_grad_(), full[1].to(device).requires_grad_()
    whole = ta.byol_contrastive_loss(o1, o2, full[2].to(device), full[3].to(device))
    whole.backward()
    split = lambda t: [p.contiguous().to(device) for p in t.split(rows)]  # noqa: E731
    p1, p2 = [p.requires_grad_() for p in split(full[0])], [p.requires_grad_() for p in split(full[1])]
    loss = ta.byol_contrastive_loss_pieces(p1, p2, split(full[2]), split(full[3]))
    loss.backward()
    assert torch.equal(loss, whole)
    assert torch.equal(torch.cat([p.grad for p in p1]), o1.grad)
    assert torch.equal(torch.cat([p.grad for p in p2]), o2.grad)
    assert rel_err(loss.item(), want) < 1e-5
    assert max_rel_to_peak(o1.grad, grads[0]) < 1e-5 and max_rel_to_peak(o2.grad, grads[1]) < 1e-5
    # argument errors: piece counts must agree, at most 8 pieces
    with pytest.raises(ValueError):
        ta.byol_contrastive_loss_pieces(p1, p2[:2], split(full[2]), split(full[3]))
    nine = [torch.randn(4, c, generator=g).to(device) for _ in range(9)]
    with pytest.raises(Exception):
        ta.byol_contrastive_loss_pieces(nine, nine, nine, nine)


def test_losses_over_a_batch_without_rows_give_nan_and_empty_gradients(device):
    """kl_div 'batchmean', cross entropy and the row means of the reference all
    divide a zero sum by zero rows: NaN loss, empty gradient, no error."""
    from argparse import Namespace

    def run(fn, *xs):
        xs = [x.clone().requires_grad_() if x.is_floating_point() else x for x in xs]
        loss = fn(*xs)
        loss.backward()
        return loss.detach().cpu(), xs[0].grad

    z, zl = torch.randn(0, 100), torch.zeros(0, dtype=torch.long)
    e, q = torch.randn(0, 128), torch.randn(0, 256)
    ns = Namespace(T=4.0, lambda_kd=0.7, kd_mode="st", moco_t=0.2)
    cases = [
        (lambda a, b: ts_oracle.kd_soft_target(a, b, 4.0), lambda a, b: ta.kd_soft_target_loss(a, b, 4.0), (z, z)),
        (lambda a, b, y: ts_oracle.soft_target_tspipe_loss(a, b, y, 4.0, 0.7),
         lambda a, b, y: ta.soft_target_tspipe_loss(a, b, y, None, ns, 0), (z, z, zl)),
        (ts_oracle.logits_mse, ta.logits_mse_loss, (z, z)),
        (ts_oracle.byol_contrastive_loss, ta.byol_contrastive_loss, (e, e, e, e)),
        (lambda a, b, c, d: ts_oracle.moco_contrastive_loss(a, b, c, d, 0.2),
         lambda a, b, c, d: ta.moco_contrastive_loss(a, b, c, d, None, ns), (q, q, q, q)),
        (lambda a, b, c, d: ts_oracle.moco_contrastive_loss(a, b, c, d, 0.2),
         lambda a, b, c, d: ta.moco_contrastive_loss(a, b, c, d, None, ns), (q.bfloat16(), ) * 4),
    ]
    for ref_fn, got_fn, xs in cases:
        ref_loss, ref_grad = run(ref_fn, *xs)
        got_loss, got_grad = run(got_fn, *[x.to(device) for x in xs])
        assert torch.isnan(ref_loss) and torch.isnan(got_loss)
        assert got_grad.shape == ref_grad.shape and got_grad.dtype == ref_grad.dtype and got_grad.is_cuda


def test_cpp_autograd_node_and_python_functions_of_the_row_losses_agree(device, monkeypatch):
    """The plain calls of the KD / squared-error / cosine / BYOL plug-ins run as a
    C++ autograd node of the host helper; it makes the same calls on the same entry
    points as the Python autograd.Functions, so loss and gradients agree bit for bit,
    also under a scaled grad_output, N-D inputs, masks and labels."""
    from tspipe_amd import _lib, losses
    if _lib.host_helper() is None or not hasattr(_lib.host_helper(), "row_loss"):
        pytest.skip("host helper not built")
    g = seeded(21)

    def both(fn, n_leaves, *xs):
        results = []
        for node in (True, False):
            monkeypatch.setattr(losses, "_HOST_NODE", node)
            leaves = [x.clone().requires_grad_() for x in xs[:n_leaves]]
            loss = fn(*leaves, *xs[n_leaves:])
            assert ("RowLossNode" in loss.grad_fn.name()) == node, loss.grad_fn.name()
            (loss * 0.37).backward()
            results.append((loss.detach(), [x.grad for x in leaves]))
        (la, ga), (lb, gb) = results
        assert bits_equal(la, lb)
        assert all(bits_equal(a, b) for a, b in zip(ga, gb))
        assert all(a.shape == x.shape for a, x in zip(ga, xs))

    for dtype in (torch.float32, torch.bfloat16):
        s = (torch.randn(6, 50, 100, generator=g) * 2).to(device, dtype)
        t = (torch.randn(6, 50, 100, generator=g) * 2).to(device, dtype)
        mask = (torch.rand(6, 50, generator=g) < 0.4).to(device)
        labels = torch.randint(0, 100, (6, 50), generator=g).to(device)
        labels[0, :7] = -100
        both(lambda a, b: ta.kd_soft_target_loss(a, b, 4.0), 1, s, t)
        both(lambda a, b: ta.distil_ce_loss(a, b, mask, 2.0, 5.0), 1, s, t)
        both(lambda a, b: ta.kd_ce_loss(a, b, labels, 2.0, 5.0, 2.0, row_mask=mask, mse_weight=0.5), 1, s, t)
        both(lambda a, b: ta.logits_mse_loss(a, b), 1, s, t)
        both(lambda a, b: ta.logits_mse_loss(a, b, mask, 0.5, False), 1, s, t)
        both(lambda a, b: ta.cosine_embedding_loss(a, b, mask, 1.5), 1, s, t)
        x = [torch.randn(77, 128, generator=g).to(device, dtype) for _ in range(4)]
        both(lambda a, b, c, d: ta.byol_contrastive_loss(a, b, c, d), 2, *x)
        both(lambda a, b: losses.regression_loss_mean(a, b), 1, x[0], x[2])
    # without gradient mode and without a leaf: a loss and nothing else
    monkeypatch.setattr(losses, "_HOST_NODE", True)
    with torch.no_grad():
        a = ta.kd_soft_target_loss(s.clone().requires_grad_(), t, 4.0)
    b = ta.kd_soft_target_loss(s, t, 4.0)
    assert a.grad_fn is None and b.grad_fn is None and bits_equal(a, b)
    # one gradient buffer per forward: a second backward is refused by either kind of node
    for node in (True, False):
        monkeypatch.setattr(losses, "_HOST_NODE", node)
        leaf = s.clone().requires_grad_()
        loss = ta.kd_soft_target_loss(leaf, t, 4.0)
        loss.backward(retain_graph=True)
        with pytest.raises(RuntimeError, match="once per forward"):
            loss.backward()
    monkeypatch.setattr(losses, "_HOST_NODE", True)
    # calls that are not plain take the Python path and its errors
    with pytest.raises(ValueError):
        ta.kd_soft_target_loss(s, t[:, :, :50], 4.0)
    with pytest.raises(TypeError):
        ta.kd_soft_target_loss(s.cpu(), t.cpu(), 4.0)
    strided = s.transpose(0, 1).requires_grad_()
    loss = ta.kd_soft_target_loss(strided, t.transpose(0, 1), 4.0)
    assert "RowLossNode" not in loss.grad_fn.name()


def test_row_losses_from_two_threads_on_two_streams(device):
    """The C++ node allocates and launches without the interpreter lock: two threads, each
    on a stream of its own, get the same bits as one thread does."""
    import threading
    g = seeded(77)
    s = (torch.randn(300, 100, generator=g) * 3).to(device)
    t = (torch.randn(300, 100, generator=g) * 3).to(device)
    y = torch.randint(0, 100, (300,), generator=g).to(device)
    x = [torch.randn(256, 128, generator=g).to(device) for _ in range(4)]

    def kd():
        leaf = s.clone().requires_grad_()
        loss = ta.kd_ce_loss(leaf, t, y, 4.0, 0.7, 1.0)
        loss.backward()
        return loss.detach(), leaf.grad

    def byol():
        a, b = x[0].clone().requires_grad_(), x[1].clone().requires_grad_()
        loss = ta.byol_contrastive_loss(a, b, x[2], x[3])
        loss.backward()
        return loss.detach(), a.grad, b.grad

    want = {"kd": kd(), "byol": byol()}
    torch.cuda.synchronize()
    got, errors = {"kd": [], "byol": []}, []

    def worker(name, fn):
        try:
            stream = torch.cuda.Stream(device)
            stream.wait_stream(torch.cuda.current_stream(device))
            with torch.cuda.stream(stream):
                for _ in range(40):
                    got[name].append(fn())
            stream.synchronize()
        except BaseException as exc:
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(n, f)) for n, f in (("kd", kd), ("byol", byol))]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    for name in got:
        assert len(got[name]) == 40
        for result in got[name]:
            assert all(bits_equal(a, b) for a, b in zip(result, want[name])), name
