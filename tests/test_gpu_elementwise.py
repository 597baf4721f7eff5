"""GPU parity: elementwise, softmax, RMSNorm, rotary, KV scatter, index_put vs the CPU oracle."""
import pytest
import torch

from oracle import cpu_fallback as oracle
from tests.parity import assert_close, assert_each, assert_exact, assert_fp32, assert_half

pytestmark = pytest.mark.gpu


def g(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1024, 4096), (3, 5, 7), (17,), (2049,), ()])
def test_add_mul_vector_and_tail(ops, dev, dtype, shape):
    a = torch.randn(shape, generator=g(0)).to(dtype)
    b = torch.randn(shape, generator=g(1)).to(dtype)
    assert_each(ops.add(a.to(dev), b.to(dev)), oracle.add(a, b))
    assert_each(ops.add(a.to(dev), b.to(dev), alpha=2), oracle.add(a, b, alpha=2))
    assert_each(ops.add(a.to(dev), b.to(dev), alpha=-0.5), oracle.add(a, b, alpha=-0.5))
    assert_each(ops.mul(a.to(dev), b.to(dev)), oracle.mul(a, b))
    assert_each(ops.sub(a.to(dev), b.to(dev), alpha=3), oracle.sub(a, b, alpha=3))
    assert_each(ops.div(a.to(dev), (b.abs() + 1).to(dev)), oracle.div(a, b.abs() + 1))


def test_broadcast_strided_mixed_and_inplace(ops, dev):
    a = torch.randn(6, 1, 33, generator=g(2))
    b = torch.randn(5, 33, generator=g(3))
    assert_each(ops.add(a.to(dev), b.to(dev)), a + b)
    at = torch.randn(40, 24, generator=g(4))
    assert_each(ops.mul(at.to(dev).t(), at.to(dev).t()[:, ::2].repeat(1, 2)), at.t() * at.t()[:, ::2].repeat(1, 2))
    # [M,N] * [N] and [M,N] * [M,1] (the decomposed RMSNorm's broadcasts)
    x = torch.randn(64, 96, generator=g(5)).bfloat16()
    w = torch.randn(96, generator=g(6)).bfloat16()
    r = torch.rand(64, 1, generator=g(7)).bfloat16()
    assert_each(ops.mul(x.to(dev), w.to(dev)), x * w)
    assert_each(ops.mul(x.to(dev), r.to(dev)), x * r)
    # type promotion is the caller's: bf16 + fp32 -> fp32 out
    assert_each(ops.add(x.to(dev), a[:, 0, :1].expand(6, 1).repeat(11, 96)[:64].to(dev)),
                 x + a[:, 0, :1].expand(6, 1).repeat(11, 96)[:64])
    # in-place variants, also on a non-contiguous destination
    y = x.clone().to(dev)
    ops.add_(y, w.to(dev), alpha=2)
    assert_each(y, x + 2 * w)
    z = at.clone().to(dev)
    ops.mul_(z.t(), at.to(dev).t())
    assert_each(z, at * at)
    # integers
    i1 = torch.randint(-100, 100, (50, 3), generator=g(8))
    i2 = torch.randint(-100, 100, (50, 3), generator=g(9))
    assert_exact(ops.add(i1.to(dev), i2.to(dev), alpha=3), i1 + 3 * i2)
    assert_exact(ops.mul(i1.int().to(dev), i2.int().to(dev)), i1.int() * i2.int())
    assert_exact(ops.div((i1 * 7).to(dev), 5, rounding_mode="floor"), torch.div(i1 * 7, 5, rounding_mode="floor"))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_column_slices_of_a_wider_matrix(ops, dev, dtype):
    """The halves of a fused gate/up projection: rows dense, row stride twice the row length, with and
    without batch dims, as inputs, as the output, in place, and as the source of a copy."""
    ffn = 1376
    gu = torch.randn(6, 40, 2 * ffn, generator=g(50)).to(dtype)
    dgu = gu.to(dev)
    for view, dview in [(gu, dgu), (gu.reshape(240, 2 * ffn), dgu.reshape(240, 2 * ffn))]:
        gate, up = view[..., :ffn], view[..., ffn:]
        dgate, dup = dview[..., :ffn], dview[..., ffn:]
        assert not dgate.is_contiguous()
        assert_each(ops.silu_mul(dgate, dup), (oracle.silu(gate).float() * up.float()).to(dtype))
        assert_each(ops.add(dgate, dup, alpha=0.5), oracle.add(gate, up, alpha=0.5))
        assert_each(ops.mul(dgate, dup), oracle.mul(gate, up))
        assert_each(ops.silu(dup), oracle.silu(up))
    # strided output (and untouched neighbours), in-place on a slice, copy out of / into a slice
    dst = torch.zeros(240, 2 * ffn, dtype=dtype, device=dev)
    a2, b2 = gu.reshape(240, 2 * ffn)[:, :ffn], gu.reshape(240, 2 * ffn)[:, ffn:]
    ops.mul(dgu.reshape(240, 2 * ffn)[:, :ffn], dgu.reshape(240, 2 * ffn)[:, ffn:], out=dst[:, ffn:])
    assert_each(dst[:, ffn:], oracle.mul(a2, b2))
    assert_exact(dst[:, :ffn], torch.zeros(240, ffn, dtype=dtype))
    work = dgu.reshape(240, 2 * ffn).clone()
    ops.add_(work[:, :ffn], work[:, ffn:])
    assert_each(work[:, :ffn], oracle.add(a2, b2))
    assert_exact(work[:, ffn:], b2)
    dense = torch.empty(240, ffn, dtype=dtype, device=dev)
    ops.copy_(dense, dgu.reshape(240, 2 * ffn)[:, ffn:])
    assert_exact(dense, b2)
    ops.copy_(dst[:, :ffn], dense)
    assert_exact(dst[:, :ffn], b2)
    # a slice whose start is not 16-byte aligned, or whose length is not a whole number of vectors, takes the generic path
    odd = dgu.reshape(240, 2 * ffn)[:, 3:3 + 1001]
    assert_each(ops.mul(odd, odd), oracle.mul(gu.reshape(240, 2 * ffn)[:, 3:3 + 1001], gu.reshape(240, 2 * ffn)[:, 3:3 + 1001]))


def test_scalar_forms(ops, dev):
    x = torch.randn(100, 3, generator=g(10))
    assert_each(ops.add(x.to(dev), 1.5), x + 1.5)
    assert_each(ops.add(x.to(dev), 2, alpha=3), x + 6)
    assert_each(ops.sub(x.to(dev), 2.0, alpha=0.5), x - 1.0)
    assert_each(ops.mul(x.to(dev), -2.5), x * -2.5)
    assert_each(ops.div(x.to(dev), 4.0), x / 4.0)
    assert_each(ops.add(x.to(dev), torch.tensor(0.25)), x + 0.25)  # CPU 0-dim tensor is peeled to a scalar
    xb = x.bfloat16()
    y = xb.clone().to(dev)
    ops.mul_(y, 3.0)
    assert_each(y, xb * 3.0)
    ops.add_(y, 1)
    assert_each(y, xb * 3.0 + 1)
    f = torch.empty(7, 9, dtype=torch.float16, device=dev)
    ops.fill_(f, 2.5)
    assert_exact(f, torch.full((7, 9), 2.5, dtype=torch.float16))
    k = torch.empty(11, dtype=torch.int64, device=dev)
    ops.fill_(k, -3)
    assert_exact(k, torch.full((11,), -3))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_unary_ops(ops, dev, dtype):
    x = torch.randn(257, 130, generator=g(11)).to(dtype)
    d = x.to(dev)
    assert_each(ops.silu(d), oracle.silu(x))
    assert_each(ops.sigmoid(d), torch.sigmoid(x.float()).to(dtype))
    assert_each(ops.neg(d), -x)
    assert_each(ops.sin(d), torch.sin(x.float()).to(dtype))
    assert_each(ops.cos(d), torch.cos(x.float()).to(dtype))
    assert_each(ops.exp(d), torch.exp(x.float()).to(dtype))
    p = (x.abs() + 0.1)
    assert_each(ops.rsqrt(p.to(dev)), torch.rsqrt(p.float()).to(dtype))
    assert_each(ops.pow(d, 2), x.float().pow(2).to(dtype))
    assert_each(ops.pow(p.to(dev), 1.7), p.float().pow(1.7).to(dtype))
    y = x.clone().to(dev)
    ops.silu_(y)
    assert_each(y, oracle.silu(x))
    u = torch.randn(257, 130, generator=g(12)).to(dtype)
    assert_each(ops.silu_mul(d, u.to(dev)), (oracle.silu(x).float() * u.float()).to(dtype))


def test_known_answers_on_device(ops, dev):
    # dipu/tests/python/unittests/test_silu.py:31-34 and test_rsqrt.py:11
    h = ops.silu(torch.ones(2, dtype=torch.half, device=dev)).float().cpu()
    f = ops.silu(torch.ones(2, device=dev)).cpu()
    assert (h - f).abs().max() < 1e-2
    x = torch.rand(10, generator=g(13))
    gold = torch.tensor([float(a) ** -0.5 for a in x])
    assert_fp32(ops.rsqrt(x.to(dev)), gold)


def test_copy_cast_cat_mean(ops, dev):
    x = torch.randn(12, 20, generator=g(14))
    d = torch.empty(20, 12, dtype=torch.bfloat16, device=dev)
    ops.copy_(d, x.to(dev).t())                      # transposed + cast
    assert_exact(d, x.t().bfloat16())
    h = torch.zeros(8, 10, device=dev)
    ops.copy_(h[::2, 1:9:2], torch.arange(16., device=dev).view(4, 4))  # hollow strides (test_copy.py:79-85)
    want = torch.zeros(8, 10)
    want[::2, 1:9:2] = torch.arange(16.).view(4, 4)
    assert_exact(h, want)
    bc = torch.empty(3, 4, 5, device=dev)
    ops.copy_(bc, torch.arange(5., device=dev))      # broadcast
    assert_exact(bc, torch.arange(5.).expand(3, 4, 5).contiguous())
    ints = torch.empty(6, dtype=torch.int32, device=dev)
    ops.copy_(ints, torch.arange(6., device=dev))    # test_cast.py:9-15: arange casts are exact
    assert_exact(ints, torch.arange(6, dtype=torch.int32))
    a, b = torch.randn(3, 4, 5, generator=g(15)), torch.randn(3, 2, 5, generator=g(16))
    assert_exact(ops.cat([a.to(dev), b.to(dev)], dim=1), torch.cat([a, b], 1))
    assert_exact(ops.cat([a.to(dev), a.to(dev)], dim=-1), torch.cat([a, a], -1))
    e = torch.empty(0)                                # 1-D empties are skipped; all of them empty: an empty result
    assert_exact(ops.cat([e.to(dev), a.to(dev), e.to(dev)], dim=2), torch.cat([e, a, e], 2))
    assert_exact(ops.cat([e.to(dev), e.to(dev)], dim=0), torch.cat([e, e], 0))
    m = torch.randn(6, 7, 64, generator=g(17))
    assert_fp32(ops.mean(m.to(dev), -1, keepdim=True), m.mean(-1, keepdim=True))
    assert_fp32(ops.mean(m.to(dev), [0, 2]), m.mean([0, 2]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_mean_over_leading_dims_and_of_long_rows(ops, dev, dtype):
    # kept dims after the reduced ones (sums down the columns, rows shared out over workgroups or not), ragged and
    # unaligned widths, and a few rows far longer than a wave's worth (a mean over everything is one such row)
    cases = [((6, 7, 64), [0]), ((6, 7, 64), [1]), ((5, 300, 24), [0, 1]), ((1000, 520), [0]), ((700, 3, 1031), [0]),
             ((4, 513, 8), [1]), ((2, 4100, 1536), [1]), ((3, 70001), [-1]), ((300, 1000), [0, 1]), ((2, 131072), [1])]
    for i, (shape, dims) in enumerate(cases):
        x = torch.randn(shape, generator=g(170 + i)).to(dtype)
        want = x.float().mean(dims)
        for keep in (False, True):
            got = ops.mean(x.to(dev), dims, keepdim=keep)
            assert got.dtype == dtype and tuple(got.shape) == tuple(x.mean(dims, keepdim=keep).shape)
            tol = 1e-5 if dtype == torch.float32 else 4e-3   # the result rounded to 16 bits
            err = (got.cpu().float().reshape(want.shape) - want).abs()
            assert bool((err <= tol * (1 + want.abs())).all()), (shape, dims, float(err.max()))
    base = torch.randn(64, 48, generator=g(190)).to(dtype)   # a strided view still goes through the dense copy
    assert (ops.mean(base.to(dev)[::2, 1:33], [0]).cpu().float() - base[::2, 1:33].float().mean(0)).abs().max() < 4e-3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_softmax(ops, dev, dtype):
    # shapes of dipu/tests/python/unittests/test_softmax.py:41-70 (dim 0 there), plus row softmax
    for shape, dim in [((256, 1000), 0), ((32, 48, 1024), 0), ((64, 4096), -1), ((2, 8, 128, 128), -1),
                       ((33, 1000), 1), ((5, 70000), -1), ((7, 3, 129), 1)]:
        x = (torch.rand(shape, generator=g(18)) * 10).to(dtype)
        assert_close(ops.softmax(x.to(dev), dim), oracle.softmax(x, dim))
    xt = torch.randn(96, 80, generator=g(19)).to(dtype)
    assert_close(ops.softmax(xt.to(dev).t(), -1), oracle.softmax(xt.t(), -1))   # non-contiguous input
    # long columns (the tiled form): ragged column blocks, masked entries, a fully masked column (NaN on both sides)
    for shape, dim in [((4100, 70), 0), ((3, 1000, 33), 1), ((128, 16), 0)]:
        x = (torch.randn(shape, generator=g(118)) * 4).to(dtype)
        x[torch.rand(shape, generator=g(119)) < 0.1] = float("-inf")
        x.select(dim, 0).fill_(1.0)                  # at least one finite entry everywhere ...
        x.movedim(dim, -1).reshape(-1, shape[dim])[5].fill_(float("-inf"))   # ... except in one column
        # (4 100 terms: stock ATen's fp32 result is itself 1.1e-5 from the float64 one here, the device's 3e-7, so the
        # fp32 case is held against the float64 computation)
        got, want = ops.softmax(x.to(dev), dim).cpu(), oracle.softmax(x.double() if dtype == torch.float32 else x, dim).to(dtype)
        assert torch.equal(got.isnan(), want.isnan())
        assert_close(got.nan_to_num(0.0), want.nan_to_num(0.0))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_softmax_and_rms_norm_short_and_long_rows(ops, dev, dtype):
    """Rows that share a wave (a few vectors each, ragged row counts), rows longer than one wave holds (a workgroup
    per row, up to 65536 16-bit elements) and rows longer than that or long and unaligned (two streaming passes:
    vocabularies of 128256 and 50257 entries, 70001 columns), with masked entries and one fully masked row in the
    softmax."""
    for rows, cols in [(1000, 64), (101, 8), (17, 24), (4099, 128), (33, 256), (300, 11008), (40, 32000), (3, 65536),
                       (5, 128256), (7, 50257), (3, 70001), (600, 16392)]:
        x = (torch.randn(rows, cols, generator=g(140)) * 3).to(dtype)
        x[torch.rand(rows, cols, generator=g(141)) < 0.05] = float("-inf")
        x[:, 0] = 0.5
        x[rows // 2].fill_(float("-inf"))
        got, want = ops.softmax(x.to(dev), -1).cpu(), oracle.softmax(x.double() if dtype == torch.float32 else x, -1).to(dtype)
        assert torch.equal(got.isnan(), want.isnan()), (rows, cols)
        assert_close(got.nan_to_num(0.0), want.nan_to_num(0.0))
        xr = torch.randn(rows, cols, generator=g(142)).to(dtype)
        w = (1 + 0.1 * torch.randn(cols, generator=g(143))).to(dtype)
        bvec = (0.1 * torch.randn(cols, generator=g(144))).to(dtype)
        inv = torch.empty(rows, dtype=torch.float32, device=dev)
        gotn = ops.rms_norm(xr.to(dev), w.to(dev), 1e-5, bias=bvec.to(dev), inv_rms=inv)
        wantn = oracle.rms_norm(xr.float(), w.float(), 1e-5) + bvec.float()
        if dtype == torch.float32:
            assert_fp32(gotn, wantn)
        else:
            assert_half(gotn, wantn)
            assert_half(ops.rms_norm(xr.to(dev), w.float().to(dev), 1e-5), oracle.rms_norm(xr.float(), w.float(), 1e-5))
        assert_fp32(inv, torch.rsqrt(xr.float().pow(2).mean(-1) + 1e-5), rel=1e-5)


def test_broadcast_rows_groups_and_mixed_dtypes(ops, dev):
    """The 8-columns-per-lane path: a bias row, a per-row scale, a table shared by every head ([b, 1, s, d] against
    [b, h, s, d]), operands of different floating dtypes, an in-place form, and a column slice as destination."""
    gq = g(130)
    x = torch.randn(2, 6, 40, 64, generator=gq).bfloat16()
    row, colv = torch.randn(64, generator=gq).bfloat16(), torch.randn(2, 6, 40, 1, generator=gq).bfloat16()
    tab = torch.randn(2, 1, 40, 64, generator=gq).bfloat16()
    f32 = torch.randn(2, 6, 40, 64, generator=gq)
    assert_each(ops.add(x.to(dev), row.to(dev), alpha=2), torch.add(x, row, alpha=2))
    assert_each(ops.mul(x.to(dev), colv.to(dev)), x * colv)
    assert_each(ops.mul(x.to(dev), tab.to(dev)), x * tab)
    assert_each(ops.sub(tab.to(dev), x.to(dev)), tab - x)                   # the broadcast operand first
    mixed = ops.add(x.to(dev), f32.to(dev))
    assert mixed.dtype == torch.float32
    assert_each(mixed, x + f32)
    assert_each(ops.div(f32.to(dev), x.half().to(dev)), f32 / x.half())
    inp = f32.clone().to(dev)
    ops.add_(inp, tab.to(dev))
    assert_each(inp, f32 + tab)
    wide = torch.zeros(2, 6, 40, 128, device=dev)
    ops.mul(f32.to(dev), row.to(dev), out=wide[..., 64:])
    assert_each(wide[..., 64:], f32 * row)
    assert float(wide[..., :64].abs().sum()) == 0.0
    # four dims that do not merge: the two halves of packed heads against a table shared by batch and heads
    # ([b, s, h, d / 2] slices of a [b, s, 3 h d] projection times [1, s, 1, d / 2]), and a permuted copy with dense rows
    qkv = torch.randn(2, 40, 3 * 6 * 64, generator=gq).bfloat16()
    q = qkv[..., : 6 * 64].reshape(2, 40, 6, 64)
    cosT = torch.randn(1, 40, 1, 32, generator=gq).bfloat16()
    dq = qkv.to(dev)[..., : 6 * 64].reshape(2, 40, 6, 64)
    assert_each(ops.mul(dq[..., 32:], cosT.to(dev)), q[..., 32:] * cosT)
    perm = torch.empty(2, 6, 40, 64, dtype=torch.bfloat16, device=dev)
    ops.copy_(perm, dq.permute(0, 2, 1, 3))
    assert_exact(perm, q.permute(0, 2, 1, 3).contiguous())
    half = torch.empty(2, 6, 40, 64, dtype=torch.float16, device=dev)
    ops.copy_(half, tab.to(dev).expand(2, 6, 40, 64))                        # broadcast copy with a cast
    assert_exact(half, tab.expand(2, 6, 40, 64).half())


def test_copy_from_a_transposed_view(ops, dev):
    """Dense destinations filled from transposed sources go through 64 x 64 tiles: ragged edges, a batch dim, 2- and
    4-byte elements, and a source whose rows are further apart than their length."""
    for shape, dt in [((130, 70), torch.bfloat16), ((64, 64), torch.float32), ((3, 100, 257), torch.float16),
                      ((1000, 33), torch.int32)]:
        src = (torch.randn(*shape[:-2], shape[-1], shape[-2] + 8, generator=g(120)) * 50).to(dt)
        view = src[..., : shape[-2]].transpose(-1, -2)          # [.., rows, cols], unit stride along rows
        dst = torch.zeros(shape, dtype=dt, device=dev)
        ops.copy_(dst, src.to(dev)[..., : shape[-2]].transpose(-1, -2))
        assert_exact(dst, view.contiguous())


def test_softmax_rows_sum_to_one_at_full_size(ops, dev):
    x = torch.randn(8192, 4096, generator=g(20)).bfloat16().to(dev)
    y = ops.softmax(x, -1)
    s = y.float().sum(-1)
    assert float((s - 1).abs().max()) < 2e-2
    assert float(y.min()) >= 0
    # order preserving within a row: the largest input holds the largest output (ties after rounding allowed)
    top = x[:64].float().argmax(-1, keepdim=True)
    assert torch.equal(y[:64].float().gather(-1, top).squeeze(-1).cpu(), y[:64].float().max(-1).values.cpu())


@pytest.mark.parametrize("dtype,eps", [(torch.float32, 1e-6), (torch.bfloat16, 1e-5), (torch.float16, 1e-5)])
def test_rms_norm(ops, dev, dtype, eps):
    for shape in [(2, 128, 512), (512, 4096), (3, 100), (4, 20000), (8, 4096), (64, 8192), (1, 2048)]:
        x = torch.randn(shape, generator=g(21)).to(dtype)
        w = (1 + 0.1 * torch.randn(shape[-1], generator=g(22))).to(dtype)
        want32 = oracle.rms_norm(x.float(), w.float(), eps)
        got = ops.rms_norm(x.to(dev), w.to(dev), eps)
        if dtype == torch.float32:
            assert_fp32(got, want32)
        else:
            assert_half(got, want32)                        # vs the fp32-computed result
            assert_half(got, oracle.rms_norm(x, w, eps))    # vs the CPU fallback in the tensor's own dtype
    x = torch.randn(37, 256, generator=g(23)).to(dtype)
    w = torch.randn(256, generator=g(24)).to(dtype)
    inv = torch.empty(37, dtype=torch.float32, device=dev)
    ops.rms_norm(x.to(dev), w.to(dev), eps, inv_rms=inv)
    assert_fp32(inv, torch.rsqrt(x.float().pow(2).mean(-1) + eps), rel=1e-5)
    # fp32 weight with a half input, and no weight at all
    if dtype != torch.float32:
        assert_half(ops.rms_norm(x.to(dev), w.float().to(dev), eps), oracle.rms_norm(x.float(), w.float(), eps))
    assert_close(ops.rms_norm(x.to(dev), None, eps), oracle.rms_norm(x.float(), torch.ones(256), eps).to(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_rotary(ops, dev, dtype):
    for seq, heads, d in [(128, 8, 64), (300, 32, 128), (16, 3, 24), (5, 2, 6)]:
        x = torch.randn(seq, heads, d, generator=g(25)).to(dtype)
        cos, sin = oracle.precompute_freqs(d, seq)
        cos, sin = cos.to(dtype), sin.to(dtype)
        want = oracle.rotary_emb(x.float(), cos.float(), sin.float())
        got = ops.rotary_emb(x.to(dev), cos.to(dev), sin.to(dev))
        (assert_fp32 if dtype == torch.float32 else assert_half)(got, want)
        # full-width tables (cos repeated), fp32 tables with a half input
        got2 = ops.rotary_emb(x.to(dev), torch.cat((cos, cos), -1).to(dev), torch.cat((sin, sin), -1).to(dev))
        assert_exact(got2, got.cpu())
        got3 = ops.rotary_emb(x.to(dev), cos.float().to(dev), sin.float().to(dev))
        (assert_fp32 if dtype == torch.float32 else assert_half)(got3, want)
        # interleaved layout (model.py:58-69) and the inverse rotation
        wi = oracle.rotary_emb_interleaved(x.float(), cos.float(), sin.float())
        gi = ops.rotary_emb(x.to(dev), cos.to(dev), sin.to(dev), interleaved=True)
        (assert_fp32 if dtype == torch.float32 else assert_half)(gi, wi)
        back = ops.rotary_emb(got, cos.to(dev), sin.to(dev), conj=True)
        if dtype == torch.float32:
            assert_fp32(back, x, rel=1e-4)
        else:
            assert_half(back, x)
    # batch broadcast: x [B, S, H, D] with tables for S positions, from a strided (split) view
    qkv = torch.randn(2, 64, 3 * 256, generator=g(26)).to(dtype)
    q = qkv.split(256, -1)[1].reshape(2, 64, 4, 64)
    cos, sin = oracle.precompute_freqs(64, 64)
    got = ops.rotary_emb(qkv.to(dev).split(256, -1)[1].reshape(2, 64, 4, 64), cos.to(dtype).to(dev), sin.to(dtype).to(dev))
    want = torch.stack([oracle.rotary_emb(q[i].float(), cos.to(dtype).float(), sin.to(dtype).float()) for i in range(2)])
    (assert_fp32 if dtype == torch.float32 else assert_half)(got, want)


def test_rotary_preserves_pair_norms_at_full_size(ops, dev, pkg):
    w = pkg.workloads.memory_bound(seed=0)
    x, cos, sin = w["rot_x"].to(dev), w["cos"].to(dev), w["sin"].to(dev)
    y = ops.rotary_emb(x, cos, sin)
    xf, yf = x.float(), y.float()
    n_in = xf[..., :64] ** 2 + xf[..., 64:] ** 2
    n_out = yf[..., :64] ** 2 + yf[..., 64:] ** 2
    assert float(((n_in - n_out).abs() / (n_in + 1e-3)).max()) < 5e-2
    assert_exact(y[0], x[0].cpu())      # position 0 is the identity, bit for bit
    back = ops.rotary_emb(y, cos, sin, conj=True)
    # two bf16 roundings and bf16 tables (cos^2 + sin^2 is 1 only to 2^-8): twice the single-op bound
    assert_half(back, x.cpu(), rel=4e-2, abs_=2e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.int8])
@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_dest_index_copy_kv_bit_exact(ops, dev, dtype, idt):
    for slots, n, heads, d in [(1000, 64, 32, 128), (50, 7, 3, 5), (9, 9, 1, 1)]:
        pool = (torch.randn(slots, heads, d, generator=g(27)) * 10).to(dtype)
        k = (torch.randn(n, heads, d, generator=g(28)) * 10).to(dtype)
        loc = torch.randperm(slots, generator=g(29))[:n].to(idt)
        want = oracle.dest_index_copy_kv(pool.clone(), k, loc)
        got = pool.clone().to(dev)
        ops.dest_index_copy_kv(k.to(dev), loc.to(dev), got)
        assert_exact(got, want)                    # written rows and every untouched slot
    # out-of-range slots are dropped, negative ones wrap like python indexing
    pool = torch.zeros(10, 2, 8, dtype=dtype)
    k = torch.ones(3, 2, 8, dtype=dtype)
    got = pool.clone().to(dev)
    ops.dest_index_copy_kv(k.to(dev), torch.tensor([3, 10, -1], dtype=idt).to(dev), got)
    want = pool.clone()
    want[3] = 1
    want[9] = 1
    assert_exact(got, want)
    # empty input
    ops.dest_index_copy_kv(torch.empty(0, 2, 8, dtype=dtype, device=dev), torch.empty(0, dtype=idt, device=dev), got)
    assert_exact(got, want)


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
def test_dest_index_copy_kv_pair_equals_two_calls(ops, dev, idt):
    """K and V rows scattered in one launch: bit-identical pools to the two single calls and to the oracle, with
    a strided source (slices of a stacked projection), a dropped out-of-range slot, rows of different length in the two
    pools (two launches inside) and an empty batch."""
    g0 = torch.Generator().manual_seed(5)
    qkv = torch.randn(37, 3 * 4 * 64, generator=g0).bfloat16()
    k, v = qkv[:, 256:512].view(37, 4, 64), qkv[:, 512:].view(37, 4, 64)
    loc = torch.randperm(500, generator=g0)[:37].to(idt)
    loc[5] = 700                                                   # outside the pool: dropped
    pk, pv = torch.randn(500, 4, 64, generator=g0).bfloat16(), torch.randn(500, 4, 64, generator=g0).bfloat16()
    keep = loc != 700
    wk, wv = pk.clone(), pv.clone()
    oracle.dest_index_copy_kv(wk, k[keep], loc[keep])
    oracle.dest_index_copy_kv(wv, v[keep], loc[keep])
    qd = qkv.to(dev)
    kd, vd = qd[:, 256:512].view(37, 4, 64), qd[:, 512:].view(37, 4, 64)
    gk, gv = pk.to(dev), pv.to(dev)
    ops.dest_index_copy_kv_pair(kd, vd, loc.to(dev), gk, gv)
    assert_exact(gk, wk)
    assert_exact(gv, wv)
    sk, sv = pk.to(dev), pv.to(dev)
    ops.dest_index_copy_kv(kd, loc.to(dev), sk)
    ops.dest_index_copy_kv(vd, loc.to(dev), sv)
    assert_exact(gk, sk.cpu())
    assert_exact(gv, sv.cpu())
    # V rows half as long as K rows
    v2, pv2 = torch.randn(37, 4, 32, generator=g0).bfloat16(), torch.zeros(500, 4, 32, dtype=torch.bfloat16)
    gk, gv2 = pk.to(dev), pv2.to(dev)
    ops.dest_index_copy_kv_pair(kd, v2.to(dev), loc.to(dev), gk, gv2)
    wv2 = pv2.clone()
    oracle.dest_index_copy_kv(wv2, v2[keep], loc[keep])
    assert_exact(gk, wk)
    assert_exact(gv2, wv2)
    # no tokens: nothing happens
    ops.dest_index_copy_kv_pair(torch.empty(0, 4, 64, dtype=torch.bfloat16, device=dev), torch.empty(0, 4, 64, dtype=torch.bfloat16, device=dev),
                                torch.empty(0, dtype=idt, device=dev), gk, gv)
    assert_exact(gk, wk)
    with pytest.raises(Exception, match="dest_loc has"):
        ops.dest_index_copy_kv_pair(kd, vd[:5], loc.to(dev), gk, gv)


def test_dest_index_copy_kv_full_pool_round_trip(ops, dev, pkg):
    w = pkg.workloads.paged_decode(seed=0, fill_pool=False)
    pool = torch.zeros_like(w["k_pool"]).to(dev)
    ops.dest_index_copy_kv(w["k_new"].to(dev), w["dest_loc"].to(dev), pool)
    assert_exact(pool[w["dest_loc"].long().to(dev)], w["k_new"])
    # exactly 64 rows of the 262144 are non-zero
    nz = (pool.view(pool.shape[0], -1) != 0).any(-1).sum().item()
    assert nz == 64


def test_index_put(ops, dev):
    # dipu/tests/python/unittests/test_index.py:78-104
    x = torch.randn(3, 4, 5, generator=g(30)).to(dev)
    idx = torch.arange(3).to(dev)
    ops.index_put_(x, [idx], torch.tensor(1.0, device=dev))
    assert_exact(x, torch.ones(3, 4, 5))
    ops.index_put_(x, [idx], torch.tensor(0.0, device=dev))
    assert_exact(x, torch.zeros(3, 4, 5))
    for shape in [(5, 4, 2, 3), (3, 4, 5), (2, 3), (10,)]:
        inp = torch.randn(shape, generator=g(31)).clamp(-3, 3) * 100
        for numel in [1, 2, 5, inp.numel() - 1]:
            if numel < 1:
                continue
            ind = [torch.randint(0, min(shape), (numel,), generator=g(32 + i)) for i in range(len(shape))]
            vals = torch.randn(numel, generator=g(40)) * 100
            want = torch.index_put(inp.clone(), ind, vals, accumulate=True)
            got = inp.clone().to(dev)
            ops.index_put_(got, [i.to(dev) for i in ind], vals.to(dev), accumulate=True)
            assert_fp32(got, want, rel=1e-4)   # assertRtolEqual's 1e-4 (common_utils.py:266-269)
    # accumulate into 16-bit floats, odd and even element offsets, a repeated row (three additions into one element)
    for dt in (torch.bfloat16, torch.float16):
        base = torch.randn(9, 7, generator=g(42)).to(dt)
        vals = torch.randn(4, 7, generator=g(43)).to(dt)
        loc = torch.tensor([8, 2, 2, 2])
        want = base.float().index_put((loc,), vals.float(), accumulate=True)
        got = base.clone().to(dev)
        ops.index_put_(got, [loc.to(dev)], vals.to(dev), accumulate=True)
        assert_half(got, want)
        assert_exact(got[[0, 1, 3, 4, 5, 6, 7]], base[[0, 1, 3, 4, 5, 6, 7]])
    # row scatter without accumulate: the KV-cache form
    pool = torch.zeros(20, 4, 8).bfloat16()
    rows = torch.randn(5, 4, 8, generator=g(41)).bfloat16()
    loc = torch.tensor([1, 19, 7, 3, 12])
    got = pool.clone().to(dev)
    ops.index_put_(got, [loc.to(dev)], rows.to(dev))
    assert_exact(got, oracle.index_put_(pool.clone(), [loc], rows))
    # the same with rows long enough for the whole-row byte mover (8 KiB, 520 bytes and 1000 bytes a row), negative
    # indices, both index types, and a value dtype that differs from the pool's (which takes the element form)
    for shape, dt in [((300, 32, 128), torch.bfloat16), ((64, 130), torch.float32), ((50, 5, 100), torch.float16)]:
        pool = torch.randn(shape, generator=g(44)).to(dt)
        loc = torch.tensor([5, -1, 17, 0, -shape[0] + 1, 33, 2])
        rows = torch.randn(len(loc), *shape[1:], generator=g(45)).to(dt)
        for idt in (torch.int64, torch.int32):
            got = pool.clone().to(dev)
            ops.index_put_(got, [loc.to(idt).to(dev)], rows.to(dev))
            assert_exact(got, oracle.index_put_(pool.clone(), [loc], rows))
        got = pool.clone().to(dev)
        ops.index_put_(got, [loc.to(dev)], rows.float().to(dev))
        assert_exact(got, oracle.index_put_(pool.clone(), [loc], rows))
