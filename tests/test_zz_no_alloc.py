"""The entry point that allocates nothing (ts_kd_fwd_bwd_static) against the
entry point it is a variant of (ts_kd_fwd_bwd), through the C ABI: two calls in
a row on the library's one scratch array, the second on a smaller input, then
a masked wide-row call, all bit-equal; and the size limit."""
import pytest
import torch

from helpers import bits_equal, seeded
from tspipe_amd import _lib

pytestmark = pytest.mark.gpu


def _both(s, t, mask, T, dev):
    lib = _lib.lib()
    rows, V = s.shape
    code = _lib.dtype_code(s.dtype)
    stream = _lib.current_stream_ptr(dev)
    mptr = None if mask is None else mask.view(torch.uint8).data_ptr()
    ws = torch.empty(lib.ts_kd_workspace_bytes(rows, V, code), dtype=torch.uint8, device=dev)
    loss_a, loss_b = torch.empty((), device=dev), torch.empty((), device=dev)
    # poisoned outputs: a kernel that skipped an element would show
    grad_a, grad_b = torch.full_like(s, 7.0), torch.full_like(s, -7.0)
    _lib.check(lib.ts_kd_fwd_bwd(s.data_ptr(), t.data_ptr(), mptr, rows, V, V, V, 1.0 / T, T * T, ws.data_ptr(),
                                 loss_a.data_ptr(), grad_a.data_ptr(), V, code, stream), "ts_kd_fwd_bwd")
    _lib.check(lib.ts_kd_fwd_bwd_static(s.data_ptr(), t.data_ptr(), mptr, rows, V, V, V, 1.0 / T, T * T,
                                        loss_b.data_ptr(), grad_b.data_ptr(), V, code, stream), "ts_kd_fwd_bwd_static")
    torch.cuda.synchronize()
    return (loss_a, grad_a), (loss_b, grad_b)


def test_static_scratch_entry_matches_workspace_entry(device):
    g = seeded(41)
    cases = [  # (rows, V, dtype, mask density or None): the second is smaller than the first
        (2048, 1000, torch.float32, None),
        (300, 100, torch.float32, None),
        (96, 30522, torch.bfloat16, 0.3),   # long masked rows: count, compaction list and row kernel in the scratch
        (64, 37, torch.float16, 0.5),
    ]
    for rows, V, dtype, density in cases:
        s = (torch.randn(rows, V, generator=g) * 3).to(dtype).to(device)
        t = (torch.randn(rows, V, generator=g) * 3).to(dtype).to(device)
        mask = None if density is None else (torch.rand(rows, generator=g) < density).to(device)
        (la, ga), (lb, gb) = _both(s, t, mask, 4.0, device)
        assert bits_equal(la.reshape(1), lb.reshape(1)), (rows, V, dtype)
        assert bits_equal(ga, gb), (rows, V, dtype)
        assert torch.isfinite(lb).item()


def test_static_scratch_entry_refuses_oversized_shapes(device):
    lib = _lib.lib()
    limit = lib.ts_kd_static_scratch_bytes()
    assert limit == 1 << 20
    rows, V = 200000, 100
    assert lib.ts_kd_workspace_bytes(rows, V, _lib.TS_F32) > limit
    x = torch.zeros(16, device=device)
    rc = lib.ts_kd_fwd_bwd_static(x.data_ptr(), x.data_ptr(), None, rows, V, V, V, 1.0, 1.0, x.data_ptr(), None, V,
                                  _lib.TS_F32, _lib.current_stream_ptr(device))
    assert rc == -5  # TS_ERR_RANGE, before anything is launched
    torch.cuda.synchronize()
