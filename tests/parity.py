"""Error metrics shared by the parity tests."""
import torch


def max_relative_error(a, b, eps=1e-6):
    """The metric of the reference's tests (test_causal_product_cpu.py:19-20)."""
    return torch.abs((a - b) / (torch.abs(a) + eps)).max().item()


def scale_error(got, want):
    """max |got - want| / max |want| per (n, h) chain, worst chain."""
    got, want = got.double(), want.double()
    num = (got - want).abs().flatten(2).max(dim=2).values
    den = want.abs().flatten(2).max(dim=2).values.clamp_min(1e-30)
    return (num / den).max().item()


def violation_fraction(got, want, rtol=1e-4, atol=1e-5):
    """Fraction of elements outside atol + rtol * |want|."""
    got, want = got.double(), want.double()
    bad = (got - want).abs() > atol + rtol * want.abs()
    return bad.double().mean().item()
