"""GPU parity: dense contractions, prefill / decode attention, int8 weight-only linear and the
fp32 decoder block vs the CPU oracle."""
import math

import pytest
import torch

from oracle import cpu_fallback as oracle
from tests.decoder import run_decoder_block, run_decomposed_decoder_block
from tests.parity import assert_close, assert_exact, assert_fp32, assert_half

pytestmark = pytest.mark.gpu


def g(seed):
    return torch.Generator().manual_seed(seed)


# ------------------------------------------------------------------ contractions
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (512, 768, 4096), (300, 200, 136), (1, 64, 64), (129, 257, 8),
                                   (1024, 1536, 512), (64, 11008, 4096)])
def test_linear_mfma_shapes(ops, dev, dtype, m, n, k):
    x = torch.randn(m, k, generator=g(0)).to(dtype)
    w = (torch.randn(n, k, generator=g(1)) * 0.05).to(dtype)
    b = torch.randn(n, generator=g(2)).to(dtype)
    want = x.float() @ w.float().t()
    assert_half(ops.linear(x.to(dev), w.to(dev)), want)
    assert_half(ops.linear(x.to(dev), w.to(dev), b.to(dev)), want + b.float())


def test_linear_known_answer_and_batched(ops, dev):
    # dipu/tests/python/unittests/test_linear.py:14-46: weight = bias = 1, x = arange
    for shape in [(3, 3), (2, 2, 3), (2, 2, 2, 3)]:
        x = torch.arange(math.prod(shape), dtype=torch.float).reshape(shape)
        y = ops.linear(x.to(dev), torch.ones(2, 3, device=dev), torch.ones(2, device=dev))
        assert_exact(y, x.sum(-1, keepdim=True).expand(*shape[:-1], 2) + 1)
    x = torch.randn(4, 96, 256, generator=g(3)).bfloat16()
    w = (torch.randn(320, 256, generator=g(4)) * 0.05).bfloat16()
    assert_half(ops.linear(x.to(dev), w.to(dev)), x.float() @ w.float().t())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_mm_bmm_matmul_addmm_baddbmm(ops, dev, dtype):
    chk = assert_fp32 if dtype == torch.float32 else assert_half
    a = torch.randn(130, 72, generator=g(5)).to(dtype)
    b = (torch.randn(72, 200, generator=g(6)) * 0.1).to(dtype)
    ref = a.float() @ b.float()
    chk(ops.mm(a.to(dev), b.to(dev)), ref)                                   # row-major mat2
    chk(ops.mm(a.to(dev), b.t().contiguous().to(dev).t()), ref)              # mat2 = W.t() view
    chk(ops.mm(a.t().contiguous().to(dev).t(), b.to(dev)), ref)              # column-major mat1
    ba = torch.randn(6, 40, 64, generator=g(7)).to(dtype)
    bb = (torch.randn(6, 64, 48, generator=g(8)) * 0.1).to(dtype)
    chk(ops.bmm(ba.to(dev), bb.to(dev)), torch.bmm(ba.float(), bb.float()))
    chk(ops.bmm(ba.to(dev), bb.transpose(1, 2).contiguous().to(dev).transpose(1, 2)), torch.bmm(ba.float(), bb.float()))
    # matmul: vector/matrix/batched/broadcast forms (test_matmul.py:8-71)
    v = torch.randn(64, generator=g(9)).to(dtype)
    chk(ops.matmul(v.to(dev), v.to(dev)), (v.float() @ v.float()))
    chk(ops.matmul(ba[0].to(dev), v.to(dev)), ba[0].float() @ v.float())
    chk(ops.matmul(v.to(dev), bb[0].to(dev)), v.float() @ bb[0].float())
    chk(ops.matmul(ba.to(dev), bb[0].to(dev)), ba.float() @ bb[0].float())
    chk(ops.matmul(ba.to(dev), bb.to(dev)), ba.float() @ bb.float())
    b4 = (torch.randn(2, 1, 64, 48, generator=g(10)) * 0.1).to(dtype)
    a4 = torch.randn(1, 3, 40, 64, generator=g(11)).to(dtype)
    chk(ops.matmul(a4.to(dev), b4.to(dev)), a4.float() @ b4.float())
    # addmm / baddbmm with broadcast addends and scalars
    c = torch.randn(200, generator=g(12)).to(dtype)
    chk(ops.addmm(c.to(dev), a.to(dev), b.to(dev), beta=0.5, alpha=2), 0.5 * c.float() + 2 * ref)
    c2 = torch.randn(130, 200, generator=g(13)).to(dtype)
    chk(ops.addmm(c2.to(dev), a.to(dev), b.to(dev)), c2.float() + ref)
    c3 = torch.randn(6, 40, 48, generator=g(14)).to(dtype)
    chk(ops.baddbmm(c3.to(dev), ba.to(dev), bb.to(dev), beta=2, alpha=0.5), 2 * c3.float() + 0.5 * torch.bmm(ba.float(), bb.float()))
    chk(ops.baddbmm(c3[:, :1].to(dev), ba.to(dev), bb.to(dev)), c3[:, :1].float() + torch.bmm(ba.float(), bb.float()))


@pytest.mark.parametrize("m,n,k,form", [
    (2048, 2048, 64, "linear"),      # 256 tiles of 128 x 128, operands straight into LDS
    (2048, 2048, 64, "mm"),          # the same with a row-major [K, N] second operand
    (200, 328, 96, "linear"),        # 64 x 64 tiles, ragged rows and columns
    (200, 328, 96, "mm"),
    (1100, 2100, 32, "addmm"),       # one stage; alpha, beta and a matrix addend in the epilogue
    (130, 200, 72, "linear"),        # K no multiple of 32: tiles staged through registers
    (130, 200, 72, "mm"),
    (136, 200, 36, "mm_at"),         # transposed first operand (row-contiguous along M)
    (2304, 2048, 40, "mm"),          # staged, 128 x 128 tiles, ragged last stage
    (64, 64, 4100, "bmm"),           # long K, batch 3
    (33, 40, 8, "linear"),           # one partial tile
    (31, 64, 64, "linear"),          # fewer than 32 rows: the FMA engine
])
def test_fp32_gemm_on_the_matrix_cores(ops, dev, m, n, k, form):
    """fp32 operands through the fp32 MFMA kernels (both tile sizes, operands straight into LDS or staged through
    registers, either layout of the second operand) against the product in float64: true fp32 products and sums, so
    only the summation order differs (1e-5 of the largest sum)."""
    x, w = torch.randn(m, k, generator=g(40)), torch.randn(n, k, generator=g(41))
    want = x.double() @ w.double().t()
    if form == "linear":
        b = torch.randn(n, generator=g(42))
        assert_fp32(ops.linear(x.to(dev), w.to(dev)), want)
        assert_fp32(ops.linear(x.to(dev), w.to(dev), b.to(dev)), want + b.double())
    elif form == "mm":
        assert_fp32(ops.mm(x.to(dev), w.t().contiguous().to(dev)), want)
    elif form == "mm_at":
        assert_fp32(ops.mm(x.t().contiguous().to(dev).t(), w.t().contiguous().to(dev)), want)
    elif form == "addmm":
        c = torch.randn(m, n, generator=g(43))
        assert_fp32(ops.addmm(c.to(dev), x.to(dev), w.to(dev).t(), beta=0.5, alpha=2), 0.5 * c.double() + 2 * want)
    else:
        xb, wb = torch.randn(3, m, k, generator=g(44)), torch.randn(3, k, n, generator=g(45))
        assert_fp32(ops.bmm(xb.to(dev), wb.to(dev)), torch.bmm(xb.double(), wb.double()))
    # a one-hot row picks one weight column exactly, whatever the tiling
    if form == "linear":
        onehot = torch.zeros(m, k)
        onehot[torch.arange(m), torch.arange(m) % k] = 1.0
        assert_exact(ops.linear(onehot.to(dev), w.to(dev)), w.t()[torch.arange(m) % k])


def test_gemm_linearity_at_7b_shapes(ops, dev):
    # size-independent property at the full prefill shape: f(x1 + x2) = f(x1) + f(x2), and a
    # one-hot row selects a weight column exactly
    w = (torch.randn(11008, 4096, generator=g(15)) * 0.02).bfloat16().to(dev)
    x1 = torch.randn(8192, 4096, generator=g(16)).bfloat16().to(dev)
    y1 = ops.linear(x1, w)
    want = x1[:32].float().cpu() @ w.float().cpu().t()
    assert_half(y1[:32], want)
    assert_half(y1[-32:], x1[-32:].float().cpu() @ w.float().cpu().t())
    onehot = torch.zeros(256, 4096, dtype=torch.bfloat16, device=dev)
    cols = torch.randint(0, 4096, (256,), generator=g(17)).to(dev)
    onehot[torch.arange(256, device=dev), cols] = 1
    assert_exact(ops.linear(onehot, w), w[:, cols].t().contiguous().cpu())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(3500, 3700, 128), (3500, 3700, 192), (3841, 3585, 320), (4096, 4096, 1088)])
def test_large_tile_gemm_edges_and_k_tile_counts(ops, dev, dtype, m, n, k):
    """At least 144 tiles of 256 x 256 and K a multiple of 64 select the 8-wave kernel whose tiles are loaded
    straight into LDS: two, three, five and seventeen K tiles (even and odd ring positions at the end),
    ragged last tile rows / columns, bias, and the alpha / beta epilogue."""
    x = torch.randn(m, k, generator=g(40)).to(dtype)
    w = (torch.randn(n, k, generator=g(41)) * 0.05).to(dtype)
    b = torch.randn(n, generator=g(42)).to(dtype)
    want = x.float() @ w.float().t()
    dx, dw = x.to(dev), w.to(dev)
    assert_half(ops.linear(dx, dw), want)
    assert_half(ops.linear(dx, dw, b.to(dev)), want + b.float())
    c = torch.randn(m, n, generator=g(43)).to(dtype)
    assert_half(ops.addmm(c.to(dev), dx, dw.t(), beta=0.5, alpha=2), 0.5 * c.float() + 2 * want)


def test_large_tile_gemm_batched_and_row_strided_operands(ops, dev):
    # 4 batches of 8 x 8 tiles; A rows taken out of a wider buffer (row stride > K), B shared by all batches
    wide = torch.randn(4, 2000, 512, generator=g(44)).bfloat16().to(dev)
    a = wide[:, :, 128:128 + 320]
    assert not a.is_contiguous()
    w = (torch.randn(1900, 320, generator=g(45)) * 0.05).bfloat16()
    want = a.float().cpu() @ w.float().t()
    assert_half(ops.matmul(a, w.to(dev).t()), want)
    bb = (torch.randn(4, 1900, 320, generator=g(46)) * 0.05).bfloat16()
    assert_half(ops.bmm(a, bb.to(dev).transpose(1, 2)), torch.bmm(a.float().cpu(), bb.float().transpose(1, 2)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("batch,m,k,n", [(1, 4096, 512, 4096),      # 256 x 256 tiles
                                         (1, 1024, 4096, 4096),     # 128 x 128 tiles
                                         (1, 200, 1024, 520),       # 128 x 128 tiles, K split, ragged edges
                                         (3, 700, 128, 136),        # batched, two K tiles, a narrow matrix
                                         (16, 2048, 2048, 128),     # the P . V product of decomposed attention
                                         (2, 2304, 192, 2048)])     # batched 256 x 256 tiles, three K tiles
def test_second_operand_read_in_place_as_k_by_n(ops, dev, dtype, batch, m, k, n):
    """mm / bmm / matmul with the right-hand side as the caller holds it, [K, N] row-major: the tile kernels read it in
    place. Checked against the fp32 product, and exactly: one-hot rows on the left select rows of the right."""
    g0 = g(91)
    a = torch.randn(batch, m, k, generator=g0).to(dtype)
    b = (torch.randn(batch, k, n, generator=g0) * 0.05).to(dtype)
    want = a.float() @ b.float()
    got = ops.bmm(a.to(dev), b.to(dev)) if batch > 1 else ops.mm(a[0].to(dev), b[0].to(dev)).unsqueeze(0)
    assert_half(got, want)
    rows = torch.randint(0, k, (batch, m), generator=g0)
    onehot = torch.zeros(batch, m, k, dtype=dtype)
    onehot.scatter_(2, rows.unsqueeze(-1), 1)
    sel = torch.gather(b, 1, rows.unsqueeze(-1).expand(batch, m, n))
    got = ops.bmm(onehot.to(dev), b.to(dev)) if batch > 1 else ops.mm(onehot[0].to(dev), b[0].to(dev)).unsqueeze(0)
    assert_exact(got, sel)
    if batch == 1:
        # a column slice of a wider matrix as the right-hand side (row stride above N), through matmul with a broadcast left side
        wide = (torch.randn(k, n + 64, generator=g0) * 0.05).to(dtype)
        a3 = torch.randn(2, m, k, generator=g0).to(dtype)
        got = ops.matmul(a3.to(dev), wide.to(dev)[:, 8:8 + n])
        assert_half(got, a3.float() @ wide[:, 8:8 + n].float())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("epilogue", ["linear", "bias", "addend", "addend_ragged", "addend_in_place_scaled", "addend_batched", "rotary",
                                      "rotary_bias", "rotary_conj", "rotary_f32_tables", "rotary_ragged_rows", "silu_mul"])
def test_four_wave_gemm_every_instantiation_exact(ops, dev, dtype, epilogue):
    """Every instantiation of the 4-wave large-tile kernel (two dtypes x plain, bias, addend (the form that finds a quarter of
    each tile's addend in LDS; also with rows and columns that end inside the last tiles and an addend with a longer row
    pitch, with the output written over the addend under alpha and beta, and batched), rotary without a bias and
    with 16-bit tables (the form whose table entries wait in LDS; also with the conjugate rotation and with rows that
    end inside the last tile), rotary with fp32 tables (the wave-uniform form), rotary with a bias (the general form)
    and gated epilogues) by name, on a problem of 288 tiles of 256 x 256 so that every workgroup walks at least one tile after
    its first (the path that requests the next tile's operands before the epilogue) and K = 256 (a prologue, one loop
    body and the tail). The kernel keeps its accumulators and operand fragments in registers the compiler only knows
    as clobbered: a change of register allocation around the loop would show here. Activations are one-hot rows, so
    every product is one weight element and the expected result is exact."""
    g0 = g(77)
    m, n, k = 8192, 2304, 256
    if epilogue in ("rotary_ragged_rows", "addend_ragged"):
        m -= 64                                         # 31 whole tile rows and 192 rows of the last one
    if epilogue == "addend_ragged":
        n -= 40                                         # 8 whole tile columns and 216 columns of the last one
    cols = torch.randint(0, k, (m,), generator=g0)
    x = torch.zeros(m, k, dtype=dtype)
    x[torch.arange(m), cols] = 1
    if epilogue == "silu_mul":
        w = torch.randn(2 * n, k, generator=g0).to(dtype)
        got = ops.linear_silu_mul(x.to(dev), w.to(dev))
        y = w.float()[:, cols].t().reshape(m, n // 32, 2, 32)
        want = (torch.nn.functional.silu(y[:, :, 0]) * y[:, :, 1]).reshape(m, n)
        assert_half(got, want)      # silu goes through exp: not an exact case, but every element is one known product
        return
    w = torch.randn(n, k, generator=g0).to(dtype)
    sel = w.float()[:, cols].t()                        # [m, n]: out[i] = w[:, cols[i]]
    if epilogue == "linear":
        assert_exact(ops.linear(x.to(dev), w.to(dev)), sel.to(dtype))
    elif epilogue == "bias":
        b = torch.randn(n, generator=g0).to(dtype)
        assert_exact(ops.linear(x.to(dev), w.to(dev), b.to(dev)), (sel + b.float()).to(dtype))
    elif epilogue == "addend":
        c = torch.randn(m, n, generator=g0).to(dtype)
        assert_exact(ops.addmm(c.to(dev), x.to(dev), w.to(dev).t()), (c.float() + sel).to(dtype))
    elif epilogue == "addend_ragged":
        wide = torch.randn(m, n + 24, generator=g0).to(dtype)      # the addend is a column slice: its rows are 24 elements apart
        got = ops.addmm(wide.to(dev)[:, 8:8 + n], x.to(dev), w.to(dev).t())
        assert_exact(got, (wide[:, 8:8 + n].float() + sel).to(dtype))
    elif epilogue == "addend_batched":
        # two batches of the same problem through baddbmm: the addend and the output of batch 1 lie a batch stride further on
        c = torch.randn(2, m, n, generator=g0).to(dtype)
        x2 = torch.stack([x, x.flip(0)])
        sel2 = torch.stack([sel, sel.flip(0)])
        got = ops.baddbmm(c.to(dev), x2.to(dev), w.to(dev).t().unsqueeze(0).expand(2, k, n))
        assert_exact(got, (c.float() + sel2).to(dtype))
    elif epilogue == "addend_in_place_scaled":
        c = torch.randn(m, n, generator=g0).to(dtype)
        dc = c.to(dev)
        got = ops.addmm(dc, x.to(dev), w.to(dev).t(), beta=0.5, alpha=2, out=dc)     # powers of two: still one rounding
        assert got.data_ptr() == dc.data_ptr()
        assert_exact(got, (0.5 * c.float() + 2 * sel).to(dtype))
    else:
        # tables of signed powers of two: each rotated value is a sum of two exactly scaled terms, rounded once
        hd, rows = 128, 64
        e = torch.randint(-3, 1, (rows, hd // 2), generator=g0).float()
        sg = torch.randint(0, 2, (rows, hd // 2), generator=g0).float() * 2 - 1
        tdt = torch.float32 if epilogue == "rotary_f32_tables" else dtype
        cos, sin = (2.0 ** e).to(tdt), (sg * 2.0 ** (e - 1)).to(tdt)
        rot = n - 2 * hd                                # the last two heads pass through, like v
        conj = epilogue == "rotary_conj"
        b = (torch.randint(-4, 5, (n,), generator=g0).float() / 4).to(dtype) if epilogue == "rotary_bias" else None
        got = ops.linear_rotary(x.to(dev), w.to(dev), cos.to(dev), sin.to(dev), rot, hd, None if b is None else b.to(dev),
                                conj=conj, interleaved=True)
        if b is not None:
            sel = sel + b.float()                       # quarters added to 8- or 11-bit values: exact in fp32
        v = sel.clone().reshape(m, n // hd, hd // 2, 2)
        cf = cos.float()[torch.arange(m) % rows][:, None, :]
        sf = sin.float()[torch.arange(m) % rows][:, None, :] * (-1.0 if conj else 1.0)
        out = torch.stack([v[..., 0] * cf - v[..., 1] * sf, v[..., 0] * sf + v[..., 1] * cf], dim=-1)
        out[:, rot // hd:] = v[:, rot // hd:]
        assert_exact(got, out.reshape(m, n).to(dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(1024, 4096, 4096), (300, 520, 1024), (65, 4096, 4096 + 64), (2047, 2048, 576),
                                   (512, 768, 4096)])
def test_split_k_gemm(ops, dev, dtype, m, n, k):
    """More than 64 rows but fewer than 144 tiles of 256 x 256, K a multiple of 64 with at least eight K tiles: the
    large-tile kernel with K split over the grid (4, 4, 13, 2 and 16 ways here; 65 K tiles in splits of 5, 9 in splits
    of 5 + 4), fp32 partial products and a reduction pass that applies bias and the alpha / beta epilogue; ragged
    last tile rows and columns."""
    x = torch.randn(m, k, generator=g(60)).to(dtype)
    w = (torch.randn(n, k, generator=g(61)) * 0.05).to(dtype)
    b = torch.randn(n, generator=g(62)).to(dtype)
    want = x.float() @ w.float().t()
    dx, dw = x.to(dev), w.to(dev)
    assert_half(ops.linear(dx, dw), want)
    assert_half(ops.linear(dx, dw, b.to(dev)), want + b.float())
    c = torch.randn(m, n, generator=g(63)).to(dtype)
    assert_half(ops.addmm(c.to(dev), dx, dw.t(), beta=0.5, alpha=2), 0.5 * c.float() + 2 * want)
    onehot = torch.zeros(m, k, dtype=dtype, device=dev)
    cols = torch.randint(0, k, (m,), generator=g(64)).to(dev)
    onehot[torch.arange(m, device=dev), cols] = 1
    assert_exact(ops.linear(onehot, dw), dw[:, cols].t().contiguous().cpu())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (5, 100, 8192 + 128), (16, 11008, 4096), (17, 4096, 11008),
                                   (40, 16 * 7 + 3, 384), (64, 16000, 128), (1, 16, 128), (64, 4096, 4096),
                                   (48, 12288, 1024 + 768), (33, 2056, 11008),
                                   (64, 12288, 4096), (33, 12296, 4096 + 128), (50, 16384, 4096 + 384), (64, 22016, 4096), (64, 9216, 4096),
                                   (64, 4096, 8192), (40, 4104, 11008), (64, 6144, 4096 + 640),
                                   (20, 8200, 640), (1, 12288, 256), (32, 32000, 384), (7, 8192, 128)])
def test_skinny_m_linear_and_addmm(ops, dev, dtype, m, n, k):
    """At most 64 rows against a K-contiguous weight with K a multiple of 128 select the weight-streaming kernel:
    one, two and four 16-column tiles per workgroup (N = 4096, 11008, 32000), K in one and in two staged chunks
    and down to a single step per wave, row groups of 16 with a ragged last group, ragged N, bias, and the
    alpha / beta epilogue with a full and a broadcast addend. With more than 32 rows K is also split over the grid
    in slices of 1024 (4, 2 with a ragged second, and 11 slices here; N = 16 * 7 + 3 is not a multiple of 8 and
    stays unsplit) and a reduction pass applies the epilogue. Five cases (more than 32 rows, at least 512
    column tiles, K from 4096) take the whole-K form with double-buffered activations: three and four tiles per
    workgroup, a last chunk of one and of three steps, a ragged last tile and a last workgroup with a tile past N;
    the three after them run it on K slices (four even slices, four with a short last one, two with a ragged
    second) that meet in the reduction pass. Weights at least 5120 columns wide (4096 at 17 to 32 rows) take the
    form that stages both operands through LDS (columns dealt evenly over the CUs, up to 64 or 128 per workgroup,
    walking K in stages of 128 from a staggered start): one to four row groups, column shares that are no multiple
    of 16, a last workgroup with fewer columns, K of one, two, three and five stages (fewer than the ring holds)
    up to 86. Two cases (more than 32 rows, 4096 and 4104 columns, K of 8192 and 11008) take that form with K split two
    ways over the grid and the reduction pass."""
    x = torch.randn(m, k, generator=g(50)).to(dtype)
    w = (torch.randn(n, k, generator=g(51)) * 0.05).to(dtype)
    b = torch.randn(n, generator=g(52)).to(dtype)
    want = x.float() @ w.float().t()
    dx, dw = x.to(dev), w.to(dev)
    assert_half(ops.linear(dx, dw), want)
    assert_half(ops.linear(dx, dw, b.to(dev)), want + b.float())
    c = torch.randn(m, n, generator=g(53)).to(dtype)
    assert_half(ops.addmm(c.to(dev), dx, dw.t(), beta=0.5, alpha=2), 0.5 * c.float() + 2 * want)
    assert_half(ops.addmm(b.to(dev), dx, dw.t()), b.float() + want)
    # a one-hot row selects a weight column exactly
    onehot = torch.zeros(m, k, dtype=dtype, device=dev)
    cols = torch.randint(0, k, (m,), generator=g(54)).to(dev)
    onehot[torch.arange(m, device=dev), cols] = 1
    assert_exact(ops.linear(onehot, dw), dw[:, cols].t().contiguous().cpu())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("m,f,k", [(4096, 3584, 256), (3700, 4000 - 32, 192), (96, 64, 80), (1, 32, 8),
                                   (5, 2048, 256), (33, 5536, 384), (48, 16384, 128), (64, 11008, 640), (20, 8224, 256)])
def test_linear_silu_mul(ops, dev, dtype, m, f, k):
    """silu(x Wg^T) * (x Wu^T) from the interleaved weight: the single-launch path (at least 144 tiles, K a
    multiple of 64, 16-bit dtypes) and the two-pass path, against the reference's four-op form in fp32. The last five
    cases (at most 64 rows, K a multiple of 128, at least 4096 stacked columns, 16-bit dtypes) take the decode-sized
    kernel with the gate applied to its sums: one to four row groups, workgroups of 64 and of 128 columns, a last
    workgroup with a single block of 64, K of one to five stages."""
    x = torch.randn(m, k, generator=g(60)).to(dtype)
    wg = (torch.randn(f, k, generator=g(61)) * 0.08).to(dtype)
    wu = (torch.randn(f, k, generator=g(62)) * 0.08).to(dtype)
    gate, up = x.float() @ wg.float().t(), x.float() @ wu.float().t()
    want = torch.nn.functional.silu(gate) * up
    w = ops.interleave_gate_up(wg.to(dev), wu.to(dev))
    assert_exact(w[32:64], wu[:32])  # block 0: 32 gate rows, then 32 up rows
    got = ops.linear_silu_mul(x.to(dev), w)
    (assert_fp32 if dtype == torch.float32 else assert_half)(got, want)
    if m >= 96:  # batch dims and a strided destination
        x3 = x[:96].reshape(2, 48, k)
        dst = torch.zeros(2, 48, 2 * f, dtype=dtype, device=dev)
        ops.linear_silu_mul(x3.to(dev), w, out=dst[..., :f])
        (assert_fp32 if dtype == torch.float32 else assert_half)(dst[..., :f], want[:96].reshape(2, 48, f))
        assert_exact(dst[..., f:], torch.zeros(2, 48, f, dtype=dtype))
    elif f >= 2048:  # the decode-sized kernel into a strided destination
        dst = torch.zeros(m, 2 * f, dtype=dtype, device=dev)
        ops.linear_silu_mul(x.to(dev), w, out=dst[:, :f])
        assert_exact(dst[:, :f], got.cpu())
        assert_exact(dst[:, f:], torch.zeros(m, f, dtype=dtype))


# ------------------------------------------------------------------ prefill attention
@pytest.mark.parametrize("dtype,table_dtype", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32)])
@pytest.mark.parametrize("m,heads,hd,vcols,k,interleaved,conj,bias", [
    (2304, 16, 128, 2048, 256, True, False, False),   # 9 x 16 tiles: one launch; q and k rotated, v through
    (2400, 57, 64, 0, 192, True, True, True),         # ragged rows and columns, all columns rotated, negative angle, bias
    (2304, 16, 128, 2048, 256, False, False, False),  # half-split pairs: projection + rotary kernel
    (40, 4, 64, 128, 128, True, False, True),         # small: projection + rotary kernel
    (64, 64, 128, 4096, 256, True, False, False),     # decode-sized, 12288 columns: the LDS-staged kernel rotates its sums (48 columns per workgroup)
    (7, 45, 128, 640, 384, True, True, True),         # one row group, 25 columns per workgroup made 26, negative angle, bias
    (33, 96, 64, 22016 - 6144, 128, True, False, True),  # 22016 columns: workgroups of 86 columns, three row groups
])
def test_linear_rotary(ops, dev, dtype, table_dtype, m, heads, hd, vcols, k, interleaved, conj, bias):
    """The stacked projection with the rotary embedding in its epilogue against the oracle's projection followed by
    the oracle's rotation (half-split: ext_ops.py:24-33; interleaved: model.py:58-69), and against this backend's
    own two separate ops."""
    rot = heads * hd
    n = rot + vcols
    x = torch.randn(m, k, generator=g(70)).to(dtype)
    w = (torch.randn(n, k, generator=g(71)) * 0.05).to(dtype)
    b = torch.randn(n, generator=g(72)).to(dtype) if bias else None
    cos, sin = oracle.precompute_freqs(hd, m)
    cos_t, sin_t = cos.to(table_dtype), sin.to(table_dtype)
    y = x.float() @ w.float().t() + (b.float() if bias else 0)
    sgn = -1.0 if conj else 1.0
    yr = y[:, :rot].reshape(m, heads, hd)
    want_rot = (oracle.rotary_emb_interleaved if interleaved else oracle.rotary_emb)(yr, cos_t.float(), sgn * sin_t.float())
    want = torch.cat([want_rot.reshape(m, rot), y[:, rot:]], dim=1)
    db = b.to(dev) if bias else None
    got = ops.linear_rotary(x.to(dev), w.to(dev), cos_t.to(dev), sin_t.to(dev), rot, hd, db, conj=conj, interleaved=interleaved)
    assert_half(got, want)
    # tables of any shape that holds [t, head_dim / 2] values are read the same way by both forms
    flat = ops.linear_rotary(x.to(dev), w.to(dev), cos_t.reshape(-1).to(dev), sin_t.reshape(-1).to(dev), rot, hd, db, conj=conj,
                             interleaved=interleaved)
    assert_exact(flat, got.cpu())
    # this backend's separate ops (one rounding more between them)
    sep = ops.linear(x.to(dev), w.to(dev), db)
    q = sep[:, :rot].view(m, heads, hd)
    ops.rotary_emb(q, cos_t.to(dev), sin_t.to(dev), conj=conj, interleaved=interleaved, out=q)
    assert_half(got, sep.float().cpu(), rel=2e-2, abs_=3e-2)   # two device results, each with its own roundings (not an oracle comparison)


def test_rotary_row_permutation_keeps_attention_scores(ops, dev):
    """A half-split checkpoint through the interleaved single-launch form: with the q / k weight rows of every head
    permuted (row 2i <- row i, row 2i + 1 <- row i + d / 2) the rotated q and k are the same permutation of the
    half-split results, so every q . k is unchanged."""
    m, heads, hd, k = 2304, 16, 128, 256
    x = torch.randn(m, k, generator=g(73)).bfloat16().to(dev)
    w = (torch.randn(2 * heads * hd, k, generator=g(74)) * 0.05).bfloat16()
    cos, sin = oracle.precompute_freqs(hd, m)
    cos, sin = cos.bfloat16().to(dev), sin.bfloat16().to(dev)
    half_split = ops.linear_rotary(x, w.to(dev), cos, sin, 2 * heads * hd, hd, interleaved=False)
    wp = ops.interleave_rotary_rows(w, hd).to(dev)
    inter = ops.linear_rotary(x, wp, cos, sin, 2 * heads * hd, hd, interleaved=True)
    perm = inter.view(m, 2 * heads, hd // 2, 2).transpose(2, 3).reshape(m, 2 * heads * hd)  # back to half-split order
    assert_half(perm, half_split.float().cpu(), rel=2e-2, abs_=3e-2)   # two device results (see above)


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 128), (torch.float16, 128), (torch.bfloat16, 64),
                                     (torch.float32, 64), (torch.float32, 40)])
def test_context_attention(ops, dev, dtype, d):
    lens = [200, 1, 130, 64, 333]
    starts, total = [], 0
    for n in lens:
        starts.append(total)
        total += n
    heads = 4
    q = torch.randn(total, heads, d, generator=g(20)).to(dtype)
    k = torch.randn(total, heads, d, generator=g(21)).to(dtype)
    v = torch.randn(total, heads, d, generator=g(22)).to(dtype)
    st, ln = torch.tensor(starts, dtype=torch.int32), torch.tensor(lens, dtype=torch.int32)
    want = oracle.context_attention(q.float(), k.float(), v.float(), st, ln)
    got = ops.context_attention(q.to(dev), k.to(dev), v.to(dev), st.to(dev), ln.to(dev), max(lens))
    (assert_fp32 if dtype == torch.float32 else assert_half)(got, want)
    # first row of every sequence equals its V row; int64 index tensors give the same result
    for s in starts:
        assert_close(got[s], v[s])
    got64 = ops.context_attention(q.to(dev), k.to(dev), v.to(dev), st.long().to(dev), ln.long().to(dev), max(lens))
    assert_exact(got64, got.cpu())


def test_context_attention_gqa_and_strided_inputs(ops, dev):
    total, heads, kvh, d = 257, 8, 2, 128
    qkv = torch.randn(total, (heads + 2 * kvh) * d, generator=g(23)).bfloat16()
    q, k, v = qkv.split([heads * d, kvh * d, kvh * d], -1)
    q, k, v = q.reshape(total, heads, d), k.reshape(total, kvh, d), v.reshape(total, kvh, d)
    st, ln = torch.tensor([0, 100]), torch.tensor([100, 157])
    want = oracle.context_attention(q.float(), k.float(), v.float(), st, ln)
    dq = qkv.to(dev).split([heads * d, kvh * d, kvh * d], -1)
    got = ops.context_attention(dq[0].reshape(total, heads, d), dq[1].reshape(total, kvh, d), dq[2].reshape(total, kvh, d),
                                st.to(dev), ln.to(dev), 157)
    assert_half(got, want)


def test_context_attention_uniform_keys_give_running_mean_at_length_2048(ops, dev):
    # property that holds at the full sequence length: identical keys -> uniform weights
    n, heads, d = 2048, 2, 128
    q = torch.randn(n, heads, d, generator=g(24)).bfloat16()
    k = torch.randn(1, heads, d, generator=g(25)).bfloat16().expand(n, -1, -1).contiguous()
    v = torch.randn(n, heads, d, generator=g(26)).bfloat16()
    got = ops.context_attention(q.to(dev), k.to(dev), v.to(dev), torch.tensor([0], dtype=torch.int32).to(dev),
                                torch.tensor([n], dtype=torch.int32).to(dev), n)
    run_mean = torch.cumsum(v.float(), 0) / torch.arange(1, n + 1).view(-1, 1, 1)
    assert_half(got, run_mean)

@pytest.mark.parametrize("heads,kvh,lens", [(8, 2, [1000, 2048, 517]), (16, 16, [1300, 90, 700]), (4, 4, [900, 1100]),
                                            (4, 2, [600, 1025, 130])])
def test_context_attention_long_ragged_batch_paired_blocks(ops, dev, heads, kvh, lens):
    """Ragged sequences up to 2048 tokens: exercises the heavy + light query-block pairing (odd and even block counts,
    sequences shorter than the longest one) and the three ways a workgroup finds its (sequence, head): a head count
    that is a multiple of 8 (one or two heads of every sequence per XCD), heads x sequences a multiple of 8, neither."""
    d = 128
    starts = [sum(lens[:i]) for i in range(len(lens))]
    total = sum(lens)
    q = torch.randn(total, heads, d, generator=g(27)).bfloat16()
    k = torch.randn(total, kvh, d, generator=g(28)).bfloat16()
    v = torch.randn(total, kvh, d, generator=g(29)).bfloat16()
    st, ln = torch.tensor(starts, dtype=torch.int32), torch.tensor(lens, dtype=torch.int32)
    want = oracle.context_attention(q.float(), k.float(), v.float(), st, ln)
    got = ops.context_attention(q.to(dev), k.to(dev), v.to(dev), st.to(dev), ln.to(dev), max(lens))
    assert_half(got, want)


@pytest.mark.parametrize("heads,kvh,d,dtype,lens", [(32, 32, 128, torch.bfloat16, [512]), (8, 2, 128, torch.bfloat16, [1000]),
                                                    (16, 4, 64, torch.float16, [700, 129, 5]), (8, 8, 128, torch.float16, [257, 256, 255, 1]),
                                                    (28, 4, 128, torch.bfloat16, [600]), (6, 3, 64, torch.bfloat16, [300, 1025])])
def test_context_attention_one_query_block_per_workgroup(ops, dev, heads, kvh, d, dtype, lens):
    """Launches too small for the paired schedule to fill the chip evenly: every 128-query block is a workgroup of its
    own, heaviest first (a single short prompt; a few ragged sequences; block counts of 4, 8, 6 and 3)."""
    starts = [sum(lens[:i]) for i in range(len(lens))]
    total = sum(lens)
    q = torch.randn(total, heads, d, generator=g(40)).to(dtype)
    k = torch.randn(total, kvh, d, generator=g(41)).to(dtype)
    v = torch.randn(total, kvh, d, generator=g(42)).to(dtype)
    st, ln = torch.tensor(starts, dtype=torch.int32), torch.tensor(lens, dtype=torch.int32)
    want = oracle.context_attention(q.float(), k.float(), v.float(), st, ln)
    got = ops.context_attention(q.to(dev), k.to(dev), v.to(dev), st.to(dev), ln.to(dev), max(lens))
    assert_half(got, want)
    assert_exact(got[starts[-1]].cpu(), v[starts[-1]].repeat_interleave(heads // kvh, dim=0))   # a sequence's first query sees one key


@pytest.mark.parametrize("heads,kvh,d,dtype,lens", [(8, 8, 96, torch.bfloat16, [300, 1, 130, 64, 333]), (8, 2, 80, torch.float16, [700, 129]),
                                                    (4, 4, 40, torch.bfloat16, [200, 513]), (4, 2, 256, torch.bfloat16, [260, 900, 64]),
                                                    (16, 16, 256, torch.float16, [1300, 2048, 517]), (8, 4, 192, torch.bfloat16, [1000]),
                                                    (32, 8, 112, torch.bfloat16, [2048, 2048])])
def test_context_attention_other_head_sizes_on_the_matrix_pipe(ops, dev, heads, kvh, d, dtype, lens):
    """Head sizes that are a multiple of 8 other than 64 and 128 take the tile layout of the next of 64 / 128 / 256, the
    pieces of a row past the head size read as zeros and never stored: sizes under 64, between 64 and 128, 256 itself
    and one between 128 and 256; both schedules (pairs of query blocks and a block per workgroup), grouped K/V heads,
    ragged batches. The neighbours of every row (the next head, the next token) hold other values, so a piece read past
    the head size would show."""
    starts = [sum(lens[:i]) for i in range(len(lens))]
    total = sum(lens)
    q = torch.randn(total, heads, d, generator=g(43)).to(dtype)
    k = torch.randn(total, kvh, d, generator=g(44)).to(dtype)
    v = torch.randn(total, kvh, d, generator=g(45)).to(dtype)
    st, ln = torch.tensor(starts, dtype=torch.int32), torch.tensor(lens, dtype=torch.int32)
    want = oracle.context_attention(q.float(), k.float(), v.float(), st, ln)
    out = torch.full((total, heads, d), 7.0, dtype=dtype, device=dev)
    got = ops.context_attention(q.to(dev), k.to(dev), v.to(dev), st.to(dev), ln.to(dev), max(lens), out=out)
    assert_half(got, want)
    assert_exact(got[starts[-1]].cpu(), v[starts[-1]].repeat_interleave(heads // kvh, dim=0))   # a sequence's first query sees one key


# ------------------------------------------------------------------ decode attention
@pytest.mark.parametrize("dtype,d,idt", [(torch.bfloat16, 128, torch.int32), (torch.float16, 64, torch.int64),
                                          (torch.float32, 64, torch.int32), (torch.bfloat16, 256, torch.int32)])
def test_token_attention_fused_and_two_call(ops, dev, pkg, dtype, d, idt):
    w = pkg.workloads.paged_decode(seed=1, batch=7, heads=4, head_dim=d, min_len=1, max_len=1300, pool_slots=8192,
                                   dtype=dtype, index_dtype=idt)
    kp, vp = w["k_pool"].clone(), w["v_pool"].clone()
    oracle.dest_index_copy_kv(kp, w["k_new"], w["dest_loc"])
    oracle.dest_index_copy_kv(vp, w["v_new"], w["dest_loc"])
    dk, dv = w["k_pool"].to(dev), w["v_pool"].to(dev)
    ops.dest_index_copy_kv(w["k_new"].to(dev), w["dest_loc"].to(dev), dk)
    ops.dest_index_copy_kv(w["v_new"].to(dev), w["dest_loc"].to(dev), dv)
    assert_exact(dk, kp)
    assert_exact(dv, vp)
    want = oracle.token_attention(w["q"].float(), kp.float(), vp.float(), w["b_loc"], w["b_seq_len"], w["max_input_len"])
    args = (w["b_loc"].to(dev), w["b_start_loc"].to(dev), w["b_seq_len"].to(dev), w["max_input_len"])
    got = ops.token_decode_attention(w["q"].to(dev), dk, dv, *args)
    chk = assert_fp32 if dtype == torch.float32 else assert_half
    chk(got, want)
    # the DIOPI two-call form: logits, then softmax . V
    att = torch.zeros(4, w["total_tokens"], dtype=torch.float32, device=dev)
    ops.token_attention(w["q"].to(dev), dk, att, *args)
    want_att = oracle.token_logits(w["q"], kp, w["b_loc"], w["b_start_loc"], w["b_seq_len"], w["max_input_len"], w["total_tokens"])
    assert_fp32(att, want_att, rel=1e-5)       # fp32 logits from either dtype: only the order of the d additions differs
    out2 = torch.empty_like(got)
    ops.token_softmax_reducev(att, dv, out2, *args)
    chk(out2, want)


@pytest.mark.parametrize("dtype,d,kvh,rep", [(torch.bfloat16, 80, 4, 2), (torch.float16, 32, 2, 1), (torch.float32, 96, 1, 4),
                                             (torch.bfloat16, 40, 8, 1), (torch.float32, 300, 2, 1)])
def test_token_attention_any_head_size(ops, dev, pkg, dtype, d, kvh, rep):
    """Head rows that are not 128, 256 or 512 bytes long: whole 16-byte pieces up to 512 bytes ride on the lanes of the
    next of those sizes with the lanes past the row's end masked (160, 64, 384 and 80 bytes here), longer rows take the
    generic kernels (1200 bytes): the fused form, the entry point that allocates nothing and the two-call form against
    the oracle (ext_ops.py:100-133), with a sequence of one token and one longer than a block of 256."""
    heads = kvh * rep
    w = pkg.workloads.paged_decode(seed=11, batch=5, heads=kvh, head_dim=d, min_len=1, max_len=700, pool_slots=4096, dtype=dtype)
    w["b_seq_len"][0] = 1                                    # b_loc is right-aligned: the last column is the token
    gq = torch.Generator().manual_seed(12)
    q = torch.randn(5, heads, d, generator=gq).to(dtype)
    want = oracle.token_attention(q.float(), w["k_pool"].float(), w["v_pool"].float(), w["b_loc"], w["b_seq_len"], w["max_input_len"])
    dk, dv = w["k_pool"].to(dev), w["v_pool"].to(dev)
    args = (w["b_loc"].to(dev), w["b_start_loc"].to(dev), w["b_seq_len"].to(dev), w["max_input_len"])
    chk = assert_fp32 if dtype == torch.float32 else assert_half
    got = ops.token_decode_attention(q.to(dev), dk, dv, *args)
    chk(got, want)
    assert_exact(ops.token_decode_attention(q.to(dev), dk, dv, *args, no_alloc=True), got.cpu())
    att = torch.zeros(heads, w["total_tokens"], dtype=torch.float32, device=dev)
    ops.token_attention(q.to(dev), dk, att, *args)
    want_att = oracle.token_logits(q, w["k_pool"], w["b_loc"], w["b_start_loc"], w["b_seq_len"], w["max_input_len"], w["total_tokens"])
    for b in range(5):                                       # only the columns of live tokens are defined
        s0, n = int(w["b_start_loc"][b]), int(w["b_seq_len"][b])
        assert_fp32(att[:, s0:s0 + n], want_att[:, s0:s0 + n], rel=1e-5)
    out2 = torch.empty_like(got)
    ops.token_softmax_reducev(att, dv, out2, *args)
    chk(out2, want)


@pytest.mark.parametrize("dtype,d,heads,kvh", [(torch.bfloat16, 96, 8, 8), (torch.float16, 112, 12, 4), (torch.bfloat16, 192, 4, 2),
                                               (torch.bfloat16, 80, 5, 5)])
def test_token_attention_masked_head_rows_over_split_sequences(ops, dev, pkg, dtype, d, heads, kvh):
    """Head sizes between the powers of two at lengths that are split into chunks and merged, on a pool whose every slot
    is in use (the lanes past a row's end must not reach past the pool's last row): four heads of a token per wave
    load, four and two query heads per K/V head, and a head count that keeps a workgroup per head."""
    w = pkg.workloads.paged_decode(seed=21, batch=9, heads=kvh, head_dim=d, min_len=700, max_len=3000, pool_slots=15285, dtype=dtype)   # exactly the tokens drawn
    gq = torch.Generator().manual_seed(22)
    q = torch.randn(9, heads, d, generator=gq).to(dtype)
    want = oracle.token_attention(q.float(), w["k_pool"].float(), w["v_pool"].float(), w["b_loc"], w["b_seq_len"], w["max_input_len"])
    dk, dv = w["k_pool"].to(dev), w["v_pool"].to(dev)
    args = (w["b_loc"].to(dev), w["b_start_loc"].to(dev), w["b_seq_len"].to(dev), w["max_input_len"])
    got = ops.token_decode_attention(q.to(dev), dk, dv, *args)
    assert_half(got, want)
    assert_exact(ops.token_decode_attention(q.to(dev), dk, dv, *args, no_alloc=True), got.cpu())
    att = torch.zeros(heads, w["total_tokens"], dtype=torch.float32, device=dev)
    ops.token_attention(q.to(dev), dk, att, *args)
    out2 = torch.empty_like(got)
    ops.token_softmax_reducev(att, dv, out2, *args)
    assert_half(out2, want)


@pytest.mark.parametrize("heads,kvh", [(8, 2), (6, 3)])
def test_token_attention_len_one_and_gqa(ops, dev, heads, kvh):
    """Grouped-query decode: four query heads per K/V head (served from one read of its rows) and two."""
    slots, d = 64, 128
    kp = torch.randn(slots, kvh, d, generator=g(30)).bfloat16()
    vp = torch.randn(slots, kvh, d, generator=g(31)).bfloat16()
    q = torch.randn(3, heads, d, generator=g(32)).bfloat16()
    lens = torch.tensor([1, 5, 1], dtype=torch.int32)
    b_loc = torch.zeros(3, 5, dtype=torch.int32)
    b_loc[0, 4] = 17
    b_loc[1] = torch.tensor([3, 60, 9, 41, 22])
    b_loc[2, 4] = 63
    starts = torch.tensor([0, 1, 6], dtype=torch.int32)
    got = ops.token_decode_attention(q.to(dev), kp.to(dev), vp.to(dev), b_loc.to(dev), starts.to(dev), lens.to(dev), 5)
    want = oracle.token_attention(q.float(), kp.float(), vp.float(), b_loc, lens, 5)
    assert_half(got, want)
    # a single cached token: the output is that token's V row for the mapped kv head
    assert_exact(got[0].cpu(), vp[17].repeat_interleave(heads // kvh, dim=0))
    assert_exact(got[2].cpu(), vp[63].repeat_interleave(heads // kvh, dim=0))


@pytest.mark.parametrize("heads,kvh,dtype,d,idt", [
    (32, 8, torch.bfloat16, 128, torch.int32),    # four query heads per K/V row read, products on packed pairs
    (16, 8, torch.float16, 64, torch.int64),      # two per read, 8 lanes per head row
    (64, 8, torch.bfloat16, 128, torch.int32),    # eight sharers: two workgroups of four per K/V head
    (8, 1, torch.float32, 64, torch.int32),       # one K/V head for all; fp32 rows take the unpacked arithmetic
    (8, 2, torch.float16, 256, torch.int32),      # 32 lanes per head row
    (12, 4, torch.bfloat16, 128, torch.int32),    # three sharers in a group with four places
    (28, 4, torch.bfloat16, 128, torch.int64),    # seven sharers: a group of four and a group of three per K/V head
    (10, 2, torch.float16, 128, torch.int32),     # five: three and two
])
def test_token_attention_grouped_query_layouts(ops, dev, heads, kvh, dtype, d, idt):
    """Fused and two-call decode attention with fewer K/V heads than query heads, over sequences of 1 to 1500 tokens
    (one to several chunks, ragged ends), against the oracle's repeat-interleaved K/V."""
    slots = 4096
    lens = [1, 1500, 777, 64, 513, 130, 1024]
    batch, width, total = len(lens), max(lens), sum(lens)
    kp = torch.randn(slots, kvh, d, generator=g(90)).to(dtype)
    vp = torch.randn(slots, kvh, d, generator=g(91)).to(dtype)
    q = torch.randn(batch, heads, d, generator=g(92)).to(dtype)
    b_loc = torch.zeros(batch, width, dtype=idt)
    for b, n in enumerate(lens):
        b_loc[b, width - n:] = torch.randint(0, slots, (n,), generator=g(93 + b)).to(idt)
    ln = torch.tensor(lens, dtype=idt)
    st = torch.zeros(batch, dtype=idt)
    st[1:] = torch.cumsum(ln, 0)[:-1]
    want = oracle.token_attention(q.float(), kp.float(), vp.float(), b_loc, ln, width)
    chk = assert_fp32 if dtype == torch.float32 else assert_half
    args = (b_loc.to(dev), st.to(dev), ln.to(dev), width)
    got = ops.token_decode_attention(q.to(dev), kp.to(dev), vp.to(dev), *args)
    chk(got, want)
    att = torch.zeros(heads, total, dtype=torch.float32, device=dev)
    ops.token_attention(q.to(dev), kp.to(dev), att, *args)
    assert_fp32(att, oracle.token_logits(q, kp, b_loc, st, ln, width, total), rel=1e-5)
    out2 = torch.empty_like(got)
    ops.token_softmax_reducev(att, vp.to(dev), out2, *args)
    chk(out2, want)
    if dtype != torch.float32:   # scores kept in the 16-bit dtype between the two calls
        att16 = torch.zeros(heads, total, dtype=dtype, device=dev)
        ops.token_attention(q.to(dev), kp.to(dev), att16, *args)
        assert_half(att16, oracle.token_logits(q, kp, b_loc, st, ln, width, total))
        out3 = torch.empty_like(got)
        ops.token_softmax_reducev(att16, vp.to(dev), out3, *args)
        assert_half(out3, want, rel=3e-2, abs_=2e-2)   # softmax of scores rounded to 8 (11) bits


# ------------------------------------------------------------------ int8 weight-only linear
@pytest.mark.parametrize("m", [1, 4, 16, 33])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_weight_only_int8_linear(ops, dev, pkg, m, dtype):
    w = pkg.workloads.int8_linear(seed=2, m=m, k=4096, n=1000, dtype=dtype)
    want = oracle.weight_only_int8_linear(w["x"], w["w"], w["scale"])
    got = ops.weight_only_int8_linear(w["x"].to(dev), w["w"].to(dev), w["scale"].to(dev))
    assert_half(got, want)
    bias = torch.randn(1000, generator=g(33)).to(dtype)
    got = ops.weight_only_int8_linear(w["x"].to(dev), w["w"].to(dev), w["scale"].float().to(dev), bias.to(dev))
    assert_half(got, want + bias.float())
    # odd K takes the scalar path
    w2 = pkg.workloads.int8_linear(seed=3, m=m, k=200, n=37, dtype=dtype)
    assert_half(ops.weight_only_int8_linear(w2["x"].to(dev), w2["w"].to(dev), w2["scale"].to(dev)),
                oracle.weight_only_int8_linear(w2["x"], w2["w"], w2["scale"]))


@pytest.mark.parametrize("m", [1, 4, 16])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_weight_only_int8_full_shape(ops, dev, pkg, m, dtype):
    """K = 4096, N = 11008 at every row count the workload names, against the oracle and against an exact case: a
    one-hot activation row selects one weight column, so the result is w * scale rounded once."""
    w = pkg.workloads.int8_linear(seed=4, m=m, k=4096, n=11008, dtype=dtype)
    got = ops.weight_only_int8_linear(w["x"].to(dev), w["w"].to(dev), w["scale"].to(dev))
    assert_half(got, oracle.weight_only_int8_linear(w["x"], w["w"], w["scale"]))
    x = torch.zeros(m, 4096, dtype=dtype)
    cols = torch.randint(0, 4096, (m,), generator=g(34))
    x[torch.arange(m), cols] = 1
    got = ops.weight_only_int8_linear(x.to(dev), w["w"].to(dev), w["scale"].to(dev))
    want = (w["w"][:, cols].float() * w["scale"].float()[:, None]).t().to(dtype)
    assert_exact(got, want)


@pytest.mark.parametrize("m,k,n", [(1, 11008, 4096), (5, 8192 + 128, 100), (37, 4096, 16 * 7 + 3), (16, 4096, 22016),
                                   (64, 4096, 4096), (100, 1024 + 256, 520), (29, 2048 + 128, 11008),
                                   (40, 2048, 11008), (20, 1024, 6200), (100, 512, 12288), (33, 768, 22016 + 8),
                                   (24, 256, 30000), (3, 256, 10240)])
def test_weight_only_int8_linear_chunked_k_row_groups_and_tile_counts(ops, dev, pkg, m, k, n):
    """K beyond one staged activation chunk (4096 columns), more than 16 rows (row groups), channel counts that leave
    partly filled workgroups, and an N large enough to use the widest workgroup. Wide weights with K a multiple of
    256 take the form that stages both operands through LDS (the last six cases, and N = 22016 above): one, two and four
    row groups, channel shares of up to 64 and up to 128 per workgroup that are no multiple of 16, more than 64 rows
    (a second workgroup row), K of one to eight stages."""
    w = pkg.workloads.int8_linear(seed=5, m=m, k=k, n=n)
    got = ops.weight_only_int8_linear(w["x"].to(dev), w["w"].to(dev), w["scale"].to(dev))
    assert_half(got, oracle.weight_only_int8_linear(w["x"], w["w"], w["scale"]))



@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(64, 14336, 4096), (33, 4096, 4096), (17, 2048 + 256, 5120), (48, 11008, 4100), (64, 2048, 200),
                                   (4, 8192, 4096), (16, 8192, 8192)])
def test_weight_only_int8_linear_narrow_weights_split_over_k(ops, dev, pkg, m, k, n, dtype):
    """Weights of fewer than 10240 channels at 17 - 64 rows, or at fewer rows with K from 8192 on: K split over workgroups
    (4, 4, 3, 3, 4, 4 and 2 slices here, one with a shorter last slice, two with a ragged last channel block), unscaled fp32 sums reduced by a second launch that applies scale and
    bias: against the oracle, with a bias in float32, and exactly on one-hot rows."""
    w = pkg.workloads.int8_linear(seed=8, m=m, k=k, n=n, dtype=dtype)
    want = oracle.weight_only_int8_linear(w["x"], w["w"], w["scale"])
    assert_half(ops.weight_only_int8_linear(w["x"].to(dev), w["w"].to(dev), w["scale"].to(dev)), want)
    bias = torch.randn(n, generator=g(37))
    assert_half(ops.weight_only_int8_linear(w["x"].to(dev), w["w"].to(dev), w["scale"].to(dev), bias.to(dev)), want + bias)
    x = torch.zeros(m, k, dtype=dtype)
    cols = torch.randint(0, k, (m,), generator=g(38))
    x[torch.arange(m), cols] = 1
    got = ops.weight_only_int8_linear(x.to(dev), w["w"].to(dev), w["scale"].to(dev))
    assert_exact(got, (w["w"][:, cols].float() * w["scale"].float()[:, None]).t().to(dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(129, 4096, 1000), (300, 1024 + 16, 520), (1024, 4096, 4096), (4608, 384, 4096),
                                   (4568, 512, 4072)])
def test_weight_only_int8_linear_many_rows(ops, dev, pkg, m, k, n, dtype):
    """From 129 rows on, without a bias, the weights are expanded once and the product goes to the dense GEMM, the
    channel scale in a pass over the result or, where the product takes the large-tile kernel (the last two shapes:
    288 tiles, the second with ragged last tiles), in that kernel's epilogue: against the oracle, with a bias (the
    streaming kernels, or that epilogue), with a float32 scale, and exactly on one-hot rows, where the result is
    w * scale (+ bias) rounded once on every route."""
    w = pkg.workloads.int8_linear(seed=6, m=m, k=k, n=n, dtype=dtype)
    want = oracle.weight_only_int8_linear(w["x"], w["w"], w["scale"])
    assert_half(ops.weight_only_int8_linear(w["x"].to(dev), w["w"].to(dev), w["scale"].to(dev)), want)
    assert_half(ops.weight_only_int8_linear(w["x"].to(dev), w["w"].to(dev), w["scale"].float().to(dev)), want)
    bias = torch.randn(n, generator=g(35)).to(dtype)
    assert_half(ops.weight_only_int8_linear(w["x"].to(dev), w["w"].to(dev), w["scale"].to(dev), bias.to(dev)), want + bias.float())
    assert_half(ops.weight_only_int8_linear(w["x"].to(dev), w["w"].to(dev), w["scale"].float().to(dev), bias.float().to(dev)),
                want + bias.float())
    x = torch.zeros(m, k, dtype=dtype)
    cols = torch.randint(0, k, (m,), generator=g(36))
    x[torch.arange(m), cols] = 1
    got = ops.weight_only_int8_linear(x.to(dev), w["w"].to(dev), w["scale"].to(dev))
    assert_exact(got, (w["w"][:, cols].float() * w["scale"].float()[:, None]).t().to(dtype))
    # and with a bias: w * scale is exact in fp32, the bias is added there, one rounding on every route
    got = ops.weight_only_int8_linear(x.to(dev), w["w"].to(dev), w["scale"].to(dev), bias.to(dev))
    assert_exact(got, ((w["w"][:, cols].float() * w["scale"].float()[:, None]).t() + bias.float()).to(dtype))


# ------------------------------------------------------------------ decoder block
def test_tiny_decoder_block_fp32_every_intermediate(ops, dev, pkg):
    x, p, cfg = pkg.workloads.tiny_block(seed=0)
    want, wi = oracle.decoder_block(x, p, cfg["heads"], cfg["eps"], cfg["theta"])
    got, gi = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg)
    for name in ["norm1", "qkv", "q_rot", "k_rot", "attn", "o", "res1", "norm2", "act", "down", "out"]:
        a, b = gi[name].cpu(), wi[name]
        assert_fp32(a.reshape(b.shape), b, rel=1e-5)
    got2, _ = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg, fused_ffn=True)
    assert_fp32(got2, want)
    # gate and up as the column halves of one stacked projection: the same numbers, op for op
    got3, gi3 = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg, fused_ffn=True, stacked_gate_up=True)
    assert_fp32(gi3["act"].cpu().reshape(wi["act"].shape), wi["act"], rel=1e-5)
    assert_fp32(got3, want)
    got4, gi4 = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg, stacked_gate_up="interleaved")
    assert_fp32(gi4["act"].cpu().reshape(wi["act"].shape), wi["act"], rel=1e-5)
    assert_fp32(got4, want)
    # rotary inside the stacked projection, on q / k weight rows permuted to the adjacent-pair convention
    got5, gi5 = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg, fused_rotary=True)
    assert_fp32(gi5["attn"].cpu().reshape(wi["attn"].shape), wi["attn"], rel=1e-5)
    assert_fp32(got5, want, rel=1e-5)


def test_small_decoder_block_bf16(ops, dev, pkg):
    x, p, cfg = pkg.workloads.llama7b_layer(seed=0, batch=2, seq=256, hidden=512, heads=4, ffn=1408)
    want, _ = oracle.decoder_block(x.float(), {k: v.float() for k, v in p.items()}, cfg["heads"], cfg["eps"], cfg["theta"])
    got, _ = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg, fused_ffn=True)
    # eleven chained bf16 roundings: 3e-2 relative / 3e-2 absolute on an O(1) output
    assert_half(got, want, rel=3e-2, abs_=3e-2)
    got, _ = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg, fused_ffn=True, stacked_gate_up=True)
    assert_half(got, want, rel=3e-2, abs_=3e-2)
    got, _ = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg, stacked_gate_up="interleaved")
    assert_half(got, want, rel=3e-2, abs_=3e-2)
    got, _ = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg, stacked_gate_up="interleaved", fused_rotary=True)
    assert_half(got, want, rel=3e-2, abs_=3e-2)


def test_decoder_block_bf16_with_both_fused_projections_in_one_launch_each(ops, dev, pkg):
    """The benchmark's configuration of the layer at a size where both fused projections take their single-launch
    form (2304 tokens, hidden 2048: 216 and 198 tiles of 256 x 256): rotary in the QKV epilogue on permuted weight
    rows, silu * mul in the gate / up epilogue, residuals through addmm-free adds."""
    x, p, cfg = pkg.workloads.llama7b_layer(seed=3, batch=3, seq=768, hidden=2048, heads=16, ffn=2816)
    want, _ = oracle.decoder_block(x.float(), {k: v.float() for k, v in p.items()}, cfg["heads"], cfg["eps"], cfg["theta"])
    got, _ = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg, stacked_gate_up="interleaved", fused_rotary=True)
    assert_half(got, want, rel=3e-2, abs_=3e-2)
    ref, _ = run_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg, fused_ffn=True)
    assert_half(got, ref.float().cpu(), rel=3e-2, abs_=3e-2)


def test_decoder_block_from_primitive_ops_only(ops, dev, pkg):
    """No fused ext op: RMSNorm, rotary tables and rotation, causal mask and attention all come from primitive
    diopi ops (pow, mean, rsqrt, arange, exp, cos, sin, cat, comparisons, masked_fill, softmax, bmm, strided copies)."""
    x, p, cfg = pkg.workloads.tiny_block(seed=1)
    want, _ = oracle.decoder_block(x, p, cfg["heads"], cfg["eps"], cfg["theta"])
    got = run_decomposed_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg)
    # the decomposed rotary tables come from exp() on the device instead of pow() on the host: 2e-5 on the tensor scale
    assert_fp32(got, want, rel=2e-5)
    x, p, cfg = pkg.workloads.llama7b_layer(seed=2, batch=2, seq=128, hidden=512, heads=4, ffn=1408)
    want, _ = oracle.decoder_block(x.float(), {k: v.float() for k, v in p.items()}, cfg["heads"], cfg["eps"], cfg["theta"])
    got = run_decomposed_decoder_block(ops, x.to(dev), {k: v.to(dev) for k, v in p.items()}, cfg)
    assert_half(got, want, rel=3e-2, abs_=3e-2)
