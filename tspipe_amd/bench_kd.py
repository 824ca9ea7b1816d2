"""Times ``ts_kd_fwd_bwd`` (soft-target KD loss, forward and backward) at chosen
shapes and checks a sample of rows against torch in fp64.

    python -m tspipe_amd.bench_kd                       # the shapes below
    python -m tspipe_amd.bench_kd 4096x30522:bf16:0.15  # rows x classes : dtype : mask density

Together with TSPIPE_AMD_LIBRARY (a measurement variant built by
``python -m tspipe_amd.build --variant NAME``) this is the A/B harness for the
KD row kernels; bench.py at the repository root times the benchmark
configurations themselves.
"""
import statistics
import sys

import torch

from . import _lib

DEFAULT_CASES = ["4096x30522:bf16:0.15", "4096x30522:bf16:0.9", "4096x30522:bf16:-", "4096x30522:f16:-",
                 "8192x4096:bf16:-", "65536x100:f32:-", "32768x1000:f32:-"]
DTYPES = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}
HBM_PEAK_GBS = 8000.0


def run(rows: int, V: int, dtype: torch.dtype, density, T: float = 2.0, samples: int = 30) -> dict:
    """One case: density None = every row carries the loss."""
    lib = _lib.lib()
    dev = torch.device("cuda", 0)
    stream = _lib.current_stream_ptr(dev)
    g = torch.Generator(device=dev).manual_seed(1)
    s = (torch.randn(rows, V, generator=g, device=dev) * 2).to(dtype)
    t = (torch.randn(rows, V, generator=g, device=dev) * 2).to(dtype)
    mask = None if density is None else (torch.rand(rows, generator=g, device=dev) < density)
    code = _lib.dtype_code(dtype)
    ws = torch.zeros(lib.ts_kd_workspace_bytes(rows, V, code), dtype=torch.uint8, device=dev)
    loss, grad = torch.empty((), device=dev), torch.full_like(s, 7.0)
    mptr = None if mask is None else mask.view(torch.uint8).data_ptr()

    def call():
        _lib.check(lib.ts_kd_fwd_bwd(s.data_ptr(), t.data_ptr(), mptr, rows, V, V, V, 1.0 / T, T * T, ws.data_ptr(),
                                     loss.data_ptr(), grad.data_ptr(), V, code, stream), "ts_kd_fwd_bwd")
    call()
    torch.cuda.synchronize()
    sel = torch.arange(rows, device=dev) if mask is None else mask.nonzero().flatten()
    n_sel = sel.numel()
    idx = sel[:: max(1, n_sel // 64)][:64]
    sd, td = s[idx].double().requires_grad_(), t[idx].double()
    ref = torch.nn.functional.kl_div(torch.log_softmax(sd / T, -1), torch.softmax(td / T, -1),
                                     reduction="sum") * T * T / max(n_sel, 1)
    ref.backward()
    grad_err = ((grad[idx].double() - sd.grad).abs().max() / sd.grad.abs().max()).item() if n_sel else 0.0
    zero_ok = True if mask is None else bool((grad[~mask] == 0).all().item())
    for _ in range(10):
        call()
    torch.cuda.synchronize()
    events = []
    for _ in range(samples):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        call()
        call()
        b.record()
        events.append((a, b))
    torch.cuda.synchronize()
    ms = statistics.median(a.elapsed_time(b) for a, b in events) / 2
    nbytes = (3 * n_sel + (rows - n_sel)) * V * s.element_size()  # read s, t + write grad; zero-fill of the rest
    return {"us": ms * 1e3, "GB/s": nbytes / ms / 1e6, "frac_hbm_peak": nbytes / ms / 1e6 / HBM_PEAK_GBS, "n_sel": n_sel,
            "loss": loss.item(), "grad_err_vs_fp64_over_peak": grad_err, "unselected_rows_zero": zero_ok}


def main(argv) -> None:
    if not torch.cuda.is_available():
        sys.exit("bench_kd: no GPU visible")
    print(f"library: {_lib.LIB_PATH}", flush=True)
    for case in argv or DEFAULT_CASES:
        shape, dt, dens = case.split(":")
        rows, V = (int(x) for x in shape.split("x"))
        print(f"{case}: ", end="", flush=True)  # names the case before its kernels run
        r = run(rows, V, DTYPES[dt], None if dens == "-" else float(dens))
        print(f"{r['us']:.1f} us, {r['GB/s']:.0f} GB/s = {r['frac_hbm_peak']:.3f} of peak, {r['n_sel']} rows with a term, "
              f"loss {r['loss']:.5f}, grad err / peak (64-row sample, fp64) {r['grad_err_vs_fp64_over_peak']:.1e}, "
              f"other rows zero: {r['unselected_rows_zero']}", flush=True)


if __name__ == "__main__":
    main(sys.argv[1:])
