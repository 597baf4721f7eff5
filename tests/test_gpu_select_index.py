"""GPU parity: where / masked_fill / tril / triu / arange / index_select / gather / comparisons vs the CPU oracle.
Pure data movement and comparisons: every check is bit-exact."""
import pytest
import torch

from oracle import cpu_fallback as oracle
from tests.parity import assert_close, assert_exact, assert_fp32

pytestmark = pytest.mark.gpu


def g(seed):
    return torch.Generator().manual_seed(seed)


def test_where_broadcast_forms(ops, dev):
    # the three shapes of dipu/tests/python/unittests/test_where.py:11-31
    x = torch.randn(3, 2, generator=g(0))
    assert_exact(ops.where(ops.gt(x.to(dev), 0), 2.0, 0.0), oracle.where(x > 0, 2.0, 0.0))
    y = torch.ones(3, 1)
    assert_exact(ops.where(ops.gt(x.to(dev), 0), x.to(dev), y.to(dev)), oracle.where(x > 0, x, y))
    x3 = torch.randn(3, 1, 1, generator=g(1))
    y3, z3 = torch.ones(3, 2, 1), torch.zeros(3, 1, 2)
    assert_exact(ops.where(ops.gt(x3.to(dev), 0), y3.to(dev), z3.to(dev)), oracle.where(x3 > 0, y3, z3))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.float64, torch.int64,
                                   torch.int32, torch.uint8, torch.bool])
def test_where_moves_every_dtype_bit_exact(ops, dev, dtype):
    a = (torch.randn(37, 65, generator=g(2)) * 100).to(dtype)
    b = (torch.randn(37, 65, generator=g(3)) * 100).to(dtype)
    c = torch.rand(37, 65, generator=g(4)) > 0.5
    assert_exact(ops.where(c.to(dev), a.to(dev), b.to(dev)), oracle.where(c, a, b))
    # non-contiguous operands and a strided destination
    out = torch.zeros(65, 37, dtype=dtype, device=dev).t()
    ops.where(c.to(dev), a.t().contiguous().to(dev).t(), b.to(dev), out=out)
    assert_exact(out, oracle.where(c, a, b))


def test_masked_fill_scalar_tensor_inplace(ops, dev):
    # shapes follow dipu/tests/python/unittests/test_masked_fill.py:8-76 at a smaller extent
    x = torch.randn(1, 1, 96, 80, generator=g(5))
    mask = torch.randn(4, 1, 96, 80, generator=g(6)).ge(0)
    assert_exact(ops.masked_fill(x.to(dev), mask.to(dev), 0), oracle.masked_fill(x, mask, 0))
    assert_exact(ops.masked_fill(x.to(dev), mask.to(dev), torch.tensor(1).to(dev)),
                 oracle.masked_fill(x, mask, torch.tensor(1)))
    assert_exact(ops.masked_fill(x.to(dev), mask.to(dev), torch.tensor(1)), oracle.masked_fill(x, mask, torch.tensor(1)))
    x4 = torch.randn(4, 1, 96, 80, generator=g(7))
    m1 = torch.randn(1, 1, 96, 80, generator=g(8)).ge(0)
    y = x4.clone().to(dev)
    ops.masked_fill_(y, m1.to(dev), 0)
    assert_exact(y, x4.clone().masked_fill_(m1, 0))
    y = x4.clone().to(dev)
    ops.masked_fill_(y, m1.to(dev), torch.tensor(1).to(dev))
    assert_exact(y, x4.clone().masked_fill_(m1, torch.tensor(1)))
    # the causal-mask idiom: scores.masked_fill(~tril(ones), -inf) on bf16
    s = torch.randn(2, 4, 33, 33, generator=g(9)).bfloat16()
    causal = torch.ones(33, 33, dtype=torch.bool).tril()
    neg = ops.eq(causal.to(dev), False)
    assert_exact(ops.masked_fill(s.to(dev), neg, float("-inf")), oracle.masked_fill(s, ~causal, float("-inf")))


def test_masked_fill_full_size(ops, dev):
    # dipu/tests/python/unittests/test_masked_fill.py:8-17 at its own size
    x = torch.randn(1, 1, 4096, 4096, generator=g(10))
    mask = torch.randn(4, 1, 4096, 4096, generator=g(11)).ge(0)
    assert_exact(ops.masked_fill(x.to(dev), mask.to(dev), 0), oracle.masked_fill(x, mask, 0))


@pytest.mark.parametrize("fn", ["tril", "triu"])
def test_triangles(ops, dev, fn):
    # dipu/tests/python/unittests/test_tri.py:9-20
    x = torch.randn(3, 3, generator=g(12))
    y = torch.randn(4, 6, generator=g(13))
    for t in (x, y, y.t(), torch.randn(2, 3, 5, 7, generator=g(14)).bfloat16(),
              torch.randint(-9, 9, (6, 4), generator=g(15))):
        for d in (0, 1, -1, 3, -4, 100, -100):
            assert_exact(getattr(ops, fn)(t.to(dev), d), getattr(oracle, fn)(t, d))
    z = y.clone().to(dev)
    ops.triu_(z, 1)
    assert_exact(z, torch.triu(y, 1))


def test_arange(ops, dev):
    # dipu/tests/python/unittests/test_arange.py:8-24
    assert_exact(ops.arange(5.0, 20.0, 1.0, device=dev), oracle.arange(5.0, 20.0, 1.0))
    assert_close(ops.arange(5.0, 20.0, 0.1, device=dev), oracle.arange(5.0, 20.0, 0.1))
    assert_exact(ops.arange(5, device=dev), torch.arange(5))
    assert_exact(ops.arange(5, 20, 1, device=dev), torch.arange(5, 20, 1))
    assert_exact(ops.arange(5.0, device=dev), torch.arange(5.0))
    assert_exact(ops.arange(10, -7, -3, device=dev), torch.arange(10, -7, -3))
    assert_exact(ops.arange(0, 8192, 1, dtype=torch.int32, device=dev), torch.arange(0, 8192, 1, dtype=torch.int32))
    assert_exact(ops.arange(0, 128, 2, dtype=torch.bfloat16, device=dev), torch.arange(0, 128, 2, dtype=torch.bfloat16))
    with pytest.raises(Exception, match="step"):
        ops.arange(0, 5, -1, dtype=torch.int64, out=torch.empty(3, dtype=torch.int64, device=dev))


def test_gather_known_answer_and_dims(ops, dev):
    # dipu/tests/python/unittests/test_gather.py:10-16
    t = torch.tensor([[1, 2], [3, 4]])
    i = torch.tensor([[0, 0], [1, 0]])
    assert_exact(ops.gather(t.to(dev), 1, i.to(dev)), torch.tensor([[1, 1], [4, 3]]))
    x = torch.randn(5, 7, 9, generator=g(16)).bfloat16()
    for dim in (0, 1, 2, -1):
        shape = [4, 6, 8]
        idx = torch.randint(0, x.shape[dim], shape, generator=g(17 + dim))
        assert_exact(ops.gather(x.to(dev), dim, idx.to(dev)), oracle.gather(x, dim, idx))
        assert_exact(ops.gather(x.to(dev), dim, idx.int().to(dev)), oracle.gather(x, dim, idx))
    # the greedy-sampling idiom: pick each row's probability at its token id
    p = torch.rand(64, 32000, generator=g(21))
    tok = torch.randint(0, 32000, (64, 1), generator=g(22))
    assert_exact(ops.gather(p.to(dev), 1, tok.to(dev)), oracle.gather(p, 1, tok))


def test_index_select_embedding_rows_and_rotary_tables(ops, dev):
    table = torch.randn(1000, 256, generator=g(23)).bfloat16()
    ids = torch.randint(0, 1000, (333,), generator=g(24))
    assert_exact(ops.index_select(table.to(dev), 0, ids.to(dev)), oracle.index_select(table, 0, ids))
    assert_exact(ops.index_select(table.to(dev), 0, ids.int().to(dev)), oracle.index_select(table, 0, ids))
    x = torch.randn(6, 10, 12, generator=g(25))
    for dim in (0, 1, 2, -2):
        idx = torch.randint(0, x.shape[dim], (7,), generator=g(26))
        assert_exact(ops.index_select(x.to(dev), dim, idx.to(dev)), oracle.index_select(x, dim, idx))
    xt = x.transpose(0, 2)
    idx = torch.tensor([11, 0, 5])
    assert_exact(ops.index_select(x.to(dev).transpose(0, 2), 0, idx.to(dev)), oracle.index_select(xt, 0, idx))
    # an index outside the table is not dereferenced: the row comes back as zeros
    bad = torch.tensor([1, 1000, -1, 2])
    got = ops.index_select(table.to(dev), 0, bad.to(dev)).cpu()
    assert_exact(got[0], table[1]), assert_exact(got[3], table[2])
    assert got[1].abs().sum() == 0 and got[2].abs().sum() == 0


@pytest.mark.parametrize("name", ["eq", "ne", "lt", "le", "gt", "ge"])
def test_comparisons(ops, dev, name):
    # dipu/tests/python/unittests/test_ge.py:14-24 for all six
    a = torch.rand(10, generator=g(27))
    b = torch.rand(10, generator=g(28))
    f = getattr(ops, name)
    assert_exact(f(a.to(dev), 3), oracle.compare(name, a, 3))
    assert_exact(f(a.to(dev), 0.5), oracle.compare(name, a, 0.5))
    assert_exact(f(a.to(dev), b.to(dev)), oracle.compare(name, a, b))
    i = torch.randint(-3, 3, (17, 5), generator=g(29))
    j = torch.randint(-3, 3, (5,), generator=g(30))
    assert_exact(f(i.to(dev), j.to(dev)), oracle.compare(name, i, j))
    assert_exact(f(i.to(dev), 0), oracle.compare(name, i, 0))
    h = torch.randn(33, 65, generator=g(31)).bfloat16()
    assert_exact(f(h.to(dev), h.t().contiguous().t().to(dev).roll(1, 0)), oracle.compare(name, h, h.roll(1, 0)))
    # position-vs-position masks: arange[:, None] >= arange[None, :]
    r = torch.arange(40)
    assert_exact(f(r.to(dev)[:, None], r.to(dev)[None, :]), oracle.compare(name, r[:, None], r[None, :]))


def test_causal_mask_from_primitives_matches_fused_attention(ops, dev):
    """The decomposed path a model written in primitive ops takes: scores = q k^T / sqrt(d), masked_fill with the
    triu mask, softmax, @ v. Must agree with the oracle's causal attention and with the fused prefill kernel."""
    B, H, S, D = 1, 4, 64, 64
    q = torch.randn(B * S, H, D, generator=g(32))
    k = torch.randn(B * S, H, D, generator=g(33))
    v = torch.randn(B * S, H, D, generator=g(34))
    qd, kd, vd = (t.to(dev).transpose(0, 1).contiguous() for t in (q, k, v))  # [H, S, D]
    scores = ops.div(ops.bmm(qd, kd.transpose(1, 2).contiguous()), D ** 0.5)
    pos = ops.arange(0, S, 1, dtype=torch.int64, device=dev)
    future = ops.gt(pos[None, :], pos[:, None])
    probs = ops.softmax(ops.masked_fill(scores, future, float("-inf")), -1)
    out = ops.bmm(probs, vd).transpose(0, 1).contiguous()
    start = torch.zeros(1, dtype=torch.int32)
    lens = torch.full((1,), S, dtype=torch.int32)
    want = oracle.context_attention(q, k, v, start, lens)
    assert_fp32(out, want)
    fused = ops.context_attention(q.to(dev), k.to(dev), v.to(dev), start.to(dev), lens.to(dev), S)
    assert_fp32(fused, want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_comparison_with_a_scalar_uses_the_tensor_dtype(ops, dev, dtype):
    """ATen rounds the scalar to the floating tensor's dtype before comparing: a tensor holding dtype(0.1) equals the
    scalar 0.1 (which it does not in double precision). Dense operands in multiples of 8 take the 8-per-lane kernel,
    the 13-element tail case the one-element kernel: both must agree with ATen."""
    for n in (4096, 13):
        x = torch.linspace(-1, 1, n).to(dtype)
        x[::3] = torch.tensor(0.1).to(dtype)
        y = x.clone()
        y[::5] += 1
        for name in ("eq", "ne", "lt", "le", "gt", "ge"):
            assert_exact(getattr(ops, name)(x.to(dev), 0.1), getattr(torch, name)(x, 0.1))
            assert_exact(getattr(ops, name)(x.to(dev), y.to(dev)), getattr(torch, name)(x, y))
    ints = torch.arange(-4, 5, dtype=torch.int32)
    assert_exact(ops.lt(ints.to(dev), 2.5), ints < 2.5)
    assert_exact(ops.eq(ints.to(dev), 3), ints == 3)


def test_index_select_blocks_and_triangles_vector_paths(ops, dev):
    """index_select whose blocks behind `dim` are whole 16-byte vectors (embedding rows; a middle dim with an outer
    one) and tril / triu with rows that are multiples of 8: the block-copy and 8-per-lane kernels, bit-exact."""
    emb = torch.randn(300, 256, generator=g(60)).bfloat16()
    idx = torch.randint(0, 300, (77,), generator=g(61))
    assert_exact(ops.index_select(emb.to(dev), 0, idx.to(dev)), emb.index_select(0, idx))
    assert_exact(ops.index_select(emb.to(dev), 0, idx.int().to(dev)), emb.index_select(0, idx))
    x3 = torch.randn(5, 40, 128, generator=g(62))
    i3 = torch.randint(0, 40, (9,), generator=g(63))
    assert_exact(ops.index_select(x3.to(dev), 1, i3.to(dev)), x3.index_select(1, i3))
    for dt in (torch.bfloat16, torch.float32, torch.int32):
        m = (torch.randn(2, 3, 70, 72, generator=g(64)) * 9).to(dt)
        for diag in (0, 1, -1, 9, -70, 100):
            assert_exact(ops.tril(m.to(dev), diag), torch.tril(m, diag))
            assert_exact(ops.triu(m.to(dev), diag), torch.triu(m, diag))
        inp = m.clone().to(dev)
        ops.triu_(inp, 1)
        assert_exact(inp, torch.triu(m, 1))


def test_masked_fill_with_a_mask_over_the_trailing_dims(ops, dev):
    """A [s, s] (or [1, 1, s, s]) mask on [b, h, s, s] scores: the condition repeats over the leading dims (the
    8-per-lane kernel indexes it modulo its length); a mask that is broadcast in the middle takes the general kernel."""
    sc = torch.randn(3, 4, 24, 40, generator=g(70)).bfloat16()
    for mshape in [(24, 40), (1, 1, 24, 40), (4, 24, 40), (3, 1, 24, 40), (40,)]:
        m = torch.rand(mshape, generator=g(71)) > 0.5
        assert_exact(ops.masked_fill(sc.to(dev), m.to(dev), float("-inf")), sc.masked_fill(m, float("-inf")))
        assert_exact(ops.where(m.to(dev), sc.to(dev), sc.neg().to(dev)), torch.where(m, sc, sc.neg()))
