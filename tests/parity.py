"""Tolerance classes of the parity gate.

  exact : index / scatter / pure moves            -> bit-identical
  fp32  : |got - want| <= 1e-5 * max(|want|, tensor scale)   (1e-5 relative)
  half  : bf16 / fp16: |got - want| <= 1e-2 + 2e-2 * |want|  (2e-2 relative / 1e-2 absolute)
"""
import torch


def assert_exact(got, want):
    assert got.dtype == want.dtype and got.shape == want.shape
    assert torch.equal(got.cpu(), want.cpu()), "not bit-identical"


def assert_fp32(got, want, rel=1e-5):
    got, want = got.detach().cpu().double(), want.detach().cpu().double()
    assert got.shape == want.shape, (got.shape, want.shape)
    scale = max(float(want.abs().max()), 1e-30) if want.numel() else 1.0
    err = (got - want).abs()
    bound = rel * torch.maximum(want.abs(), torch.full_like(want, scale))
    bad = err > bound
    assert not bool(bad.any()), f"max err {float(err.max()):.3e} vs scale {scale:.3e}; {int(bad.sum())} elements out of tolerance"


def assert_half(got, want, rel=2e-2, abs_=1e-2):
    got, want = got.detach().cpu().double(), want.detach().cpu().double()
    assert got.shape == want.shape, (got.shape, want.shape)
    err = (got - want).abs()
    bad = err > abs_ + rel * want.abs()
    assert not bool(bad.any()), f"max err {float(err.max()):.3e}; {int(bad.sum())} of {want.numel()} elements out of tolerance"


def assert_close(got, want):
    if want.dtype in (torch.float16, torch.bfloat16) or got.dtype in (torch.float16, torch.bfloat16):
        assert_half(got, want)
    elif want.dtype.is_floating_point:
        assert_fp32(got, want)
    else:
        assert_exact(got, want)
