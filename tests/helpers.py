"""Shared input generators and comparison helpers for the parity tests."""
import torch


def seeded(seed: int) -> torch.Generator:
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def param_lists(shapes, seed: int, std: float = 0.02):
    """teacher, student: independent N(0, std) fp32 tensors of the given shapes (CPU)."""
    g = seeded(seed)
    teacher = [torch.randn(s, generator=g) * std for s in shapes]
    student = [torch.randn(s, generator=g) * std for s in shapes]
    return teacher, student


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    if a.dim() == 0:
        a, b = a.reshape(1), b.reshape(1)
    return bool(torch.equal(a.view(torch.uint8), b.view(torch.uint8)))


def max_rel_to_peak(x: torch.Tensor, ref: torch.Tensor) -> float:
    """max|x - ref| / max|ref|, in fp64."""
    x, ref = x.detach().cpu().double(), ref.detach().cpu().double()
    peak = ref.abs().max().item()
    return (x - ref).abs().max().item() / (peak if peak > 0 else 1.0)


def rel_err(x, ref) -> float:
    x, ref = float(x), float(ref)
    return abs(x - ref) / (abs(ref) if ref != 0 else 1.0)
