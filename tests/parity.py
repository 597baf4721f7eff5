"""Tolerance classes of the parity gate.

  exact : index / scatter / pure moves            -> bit-identical
  fp32  : contractions and row reductions (GEMM, attention, softmax, RMSNorm, mean): |got - want| <= 1e-5 *
          max(|want|, tensor scale), "1e-5 relative" read on the scale of the tensor, because an output element that
          is the small difference of large terms carries the rounding of those terms, whatever adds them up;
          elementwise ops (assert_each): per element, |got - want| <= 1e-5 * |want| + 1e-7 (the floor is one fp32 ulp
          at 1.0, for results next to a zero crossing)
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


def assert_fp32_each(got, want, rel=1e-5, floor=1e-7):
    got, want = got.detach().cpu().double(), want.detach().cpu().double()
    assert got.shape == want.shape, (got.shape, want.shape)
    err = (got - want).abs()
    bad = err > rel * want.abs() + floor
    assert not bool(bad.any()), f"max err {float(err.max()):.3e}; {int(bad.sum())} of {want.numel()} elements out of tolerance"


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


def assert_each(got, want):
    """assert_close for elementwise ops: fp32 is held per element, not on the tensor's scale."""
    if want.dtype == torch.float32 and got.dtype == torch.float32:
        assert_fp32_each(got, want)
    else:
        assert_close(got, want)
