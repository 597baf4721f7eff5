"""Seeded random sweeps over the op families, each case against the CPU oracle (stock ATen on the same inputs, or the
restated spec functions): many more shapes, dtypes, strides and routes than the hand-picked cases hold. A failing
case is reported with everything needed to replay it (seed, case number, shapes)."""
import random

import pytest
import torch

from oracle import cpu_fallback as oracle
from tests.parity import assert_close, assert_each, assert_exact, assert_fp32, assert_half

pytestmark = pytest.mark.gpu

FLOATS = [torch.bfloat16, torch.float16, torch.float32]
INTS = [torch.int32, torch.int64, torch.int16, torch.uint8, torch.int8]


def _report(failed, n):
    assert not failed, f"{len(failed)} of {n} cases failed:\n" + "\n".join(failed[:20])


@pytest.mark.parametrize("seed,n", [(1, 120), (2, 120)])
def test_sweep_gemm(ops, dev, seed, n):
    """linear (+bias, strided), addmm, mm, the gated linear and the int8 weight-only linear over the shapes that choose
    between the large-tile, 128-tile, split-K and the decode-sized kernels."""
    rng = random.Random(seed)
    pick = rng.choice
    Ms = [1, 2, 3, 7, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 100, 128, 129, 200, 255, 256, 257, 300, 511, 513, 700, 1024, 1500]
    Ks = [8, 24, 64, 72, 128, 136, 192, 256, 320, 384, 512, 640, 1000, 1024, 2048, 2752, 4096, 4104, 5504, 8192, 11008]
    Ns = [8, 16, 24, 40, 64, 128, 136, 256, 264, 512, 1000, 1024, 2048, 4096, 4104, 5120, 6144, 8192, 8200, 10240, 11008, 12288, 16384, 22016, 32000]
    failed = []
    for case in range(n):
        kind = pick(["linear", "linear", "linear_bias", "addmm", "mm", "silu", "w8", "w8_bias", "linear_strided"])
        dtype = pick([torch.bfloat16, torch.bfloat16, torch.float16])
        m, k, nn = pick(Ms), pick(Ks), pick(Ns)
        if m * k * nn > 2e10: m = max(1, int(2e10 / (k * nn)))
        g = torch.Generator().manual_seed(seed * 100003 + case)
        desc = f"case {case} {kind} {dtype} m={m} k={k} n={nn}"
        x = torch.randn(m, k, generator=g).to(dtype)
        try:
            if kind in ("w8", "w8_bias"):
                w = torch.randint(-127, 128, (nn, k), generator=g, dtype=torch.int8)
                sc = (torch.rand(nn, generator=g) * 0.019 + 0.001).to(dtype)
                b = torch.randn(nn, generator=g).to(dtype) if kind == "w8_bias" else None
                want = x.float() @ (w.float() * sc.float()[:, None]).t() + (b.float() if b is not None else 0)
                got = ops.weight_only_int8_linear(x.to(dev), w.to(dev), sc.to(dev), b.to(dev) if b is not None else None)
                # products are exact in fp32 and summed in fp32 on both sides: per element, 2e-2 relative / 1e-2 absolute
                assert_half(got, want)
            elif kind == "silu":
                f = max(32, (nn // 2) // 32 * 32)
                w = (torch.randn(2 * f, k, generator=g) * 0.05).to(dtype)
                y = x.float() @ w.float().t()
                y = y.reshape(m, f // 32, 2, 32)
                want = (torch.nn.functional.silu(y[:, :, 0]) * y[:, :, 1]).reshape(m, f)
                got = ops.linear_silu_mul(x.to(dev), w.to(dev))
                assert_half(got, want)
            else:
                w = (torch.randn(nn, k, generator=g) * 0.05).to(dtype)
                if kind == "linear":
                    want = x.float() @ w.float().t()
                    got = ops.linear(x.to(dev), w.to(dev))
                elif kind == "linear_bias":
                    b = torch.randn(nn, generator=g).to(dtype)
                    want = x.float() @ w.float().t() + b.float()
                    got = ops.linear(x.to(dev), w.to(dev), b.to(dev))
                elif kind == "linear_strided":
                    xs = torch.randn(m, k + 8, generator=g).to(dtype)
                    dst = torch.zeros(m, nn + 16, dtype=dtype, device=dev)
                    xd = xs.to(dev)[:, :k]
                    want = xs[:, :k].float() @ w.float().t()
                    ops.linear(xd, w.to(dev), out=dst[:, :nn])
                    got = dst[:, :nn]
                    assert float(dst[:, nn:].abs().max()) == 0.0, "wrote past the destination view"
                elif kind == "addmm":
                    c = torch.randn(m, nn, generator=g).to(dtype)
                    beta, alpha = pick([1, 0.5, 2]), pick([1, 0.25])
                    want = beta * c.float() + alpha * (x.float() @ w.float().t())
                    got = ops.addmm(c.to(dev), x.to(dev), w.to(dev).t(), beta=beta, alpha=alpha)
                else:
                    wt = w.t().contiguous()   # [k, n] row-major second operand
                    want = x.float() @ wt.float()
                    got = ops.mm(x.to(dev), wt.to(dev))
                assert_half(got, want)
        except AssertionError as e:
            failed.append(desc + ": " + str(e)[:200])
    _report(failed, n)


@pytest.mark.parametrize("seed,n", [(1, 80), (2, 80)])
def test_sweep_gemm_fp32(ops, dev, seed, n):
    """fp32 products (linear with and without bias, into a strided destination, addmm, mm with either operand layout,
    bmm) over shapes on both sides of what the matrix-core kernel takes (multiples of 4 along the contiguous
    dims, at least 32 rows and columns) and its two tile sizes, against the product in float64: true fp32
    multiplies and adds, so the error is that of the summation order, a few 1e-7 of the scale of the terms."""
    rng = random.Random(seed)
    pick = rng.choice
    Ms = [1, 4, 31, 32, 33, 36, 63, 64, 65, 100, 128, 132, 200, 256, 300, 512, 700, 1024, 2048]
    Ks = [4, 8, 12, 16, 20, 30, 64, 72, 100, 128, 250, 256, 512, 1000, 1024, 2048, 4096]
    Ns = [8, 32, 36, 40, 64, 100, 128, 130, 136, 256, 512, 1000, 1024, 2048, 4096, 4100]
    failed = []
    for case in range(n):
        kind = pick(["linear", "linear_bias", "linear_strided", "addmm", "mm", "mm_at", "bmm"])
        m, k, nn = pick(Ms), pick(Ks), pick(Ns)
        if m * k * nn > 3e9: m = max(1, int(3e9 / (k * nn)))
        g = torch.Generator().manual_seed(seed * 7919 + case)
        desc = f"case {case} {kind} m={m} k={k} n={nn}"
        try:
            if kind == "bmm":
                bt = pick([1, 3, 8])
                m, nn, k = min(m, 256), min(nn, 256), min(k, 512)
                a, b = torch.randn(bt, m, k, generator=g), torch.randn(bt, k, nn, generator=g)
                want = torch.bmm(a.double(), b.double())
                got = ops.bmm(a.to(dev), b.to(dev))
            else:
                x, w = torch.randn(m, k, generator=g), torch.randn(nn, k, generator=g)
                want = x.double() @ w.double().t()
                if kind == "linear":
                    got = ops.linear(x.to(dev), w.to(dev))
                elif kind == "linear_bias":
                    b = torch.randn(nn, generator=g)
                    want = want + b.double()
                    got = ops.linear(x.to(dev), w.to(dev), b.to(dev))
                elif kind == "linear_strided":
                    pad = pick([4, 8, 3])
                    xs = torch.randn(m, k + pad, generator=g)
                    dst = torch.zeros(m, nn + pad, device=dev)
                    want = xs[:, :k].double() @ w.double().t()
                    ops.linear(xs.to(dev)[:, :k], w.to(dev), out=dst[:, :nn])
                    got = dst[:, :nn]
                    assert float(dst[:, nn:].abs().max()) == 0.0, "wrote past the destination view"
                elif kind == "addmm":
                    c = torch.randn(m, nn, generator=g)
                    beta, alpha = pick([1, 0.5, 2]), pick([1, 0.25])
                    want = beta * c.double() + alpha * want
                    got = ops.addmm(c.to(dev), x.to(dev), w.to(dev).t(), beta=beta, alpha=alpha)
                elif kind == "mm":
                    got = ops.mm(x.to(dev), w.t().contiguous().to(dev))           # [k, n] row-major second operand
                else:
                    got = ops.mm(x.t().contiguous().to(dev).t(), w.to(dev).t())   # column-major first operand
            # terms of magnitude ~1, sums of magnitude ~sqrt(k): 1e-5 of the largest sum
            assert_fp32(got, want, rel=1e-5)
        except AssertionError as e:
            failed.append(desc + ": " + str(e)[:200])
    _report(failed, n)


@pytest.mark.parametrize("seed,n", [(1, 150), (2, 150)])
def test_sweep_attention(ops, dev, pkg, seed, n):
    """Prefill over ragged packed sequences (gaps between them, empty ones) and decode over a paged pool (fused, without
    allocation), any head size, grouped kv heads, int32 / int64 tables."""
    rng = random.Random(seed)
    failed = []
    for case in range(n):
        kind = rng.choice(["prefill", "prefill", "decode", "decode", "decode_noalloc"])
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        d = rng.choice([64, 128, 128, 128, 32, 80])
        kvh = rng.choice([1, 2, 4, 8])
        heads = kvh * rng.choice([1, 1, 2, 4])
        idt = rng.choice([torch.int32, torch.int64])
        g = torch.Generator().manual_seed(seed * 7919 + case)
        desc = f"case {case} {kind} {dtype} heads={heads}/{kvh} d={d} idx={idt}"
        try:
            if kind == "prefill":
                batch = rng.choice([1, 2, 3, 5])
                maxl = rng.choice([1, 17, 64, 127, 128, 129, 255, 257, 500, 1000])
                if dtype == torch.float32 or d not in (64, 128): maxl = min(maxl, 257)   # scalar kernel: one workgroup per query
                lens = [rng.randint(0 if batch > 1 else 1, maxl) for _ in range(batch)]
                gaps = [rng.choice([0, 0, 3]) for _ in range(batch)]
                starts, off = [], 0
                for L, gp in zip(lens, gaps):
                    off += gp
                    starts.append(off)
                    off += L
                tokens = max(off, 1)
                desc += f" lens={lens} starts={starts}"
                q = torch.randn(tokens, heads, d, generator=g).to(dtype)
                k = torch.randn(tokens, kvh, d, generator=g).to(dtype)
                v = torch.randn(tokens, kvh, d, generator=g).to(dtype)
                st, ln = torch.tensor(starts, dtype=idt), torch.tensor(lens, dtype=idt)
                want = oracle.context_attention(q, k, v, st, ln)
                out = torch.zeros_like(q).to(dev)
                ops.context_attention(q.to(dev), k.to(dev), v.to(dev), st.to(dev), ln.to(dev), max(max(lens), 1), out=out)
                got = out.cpu()
                mask = torch.zeros(tokens, dtype=torch.bool)
                for s, L in zip(starts, lens): mask[s:s + L] = True
                (assert_fp32 if dtype == torch.float32 else assert_half)(got[mask], want[mask])
                assert float(got[~mask].abs().sum()) == 0.0, "rows outside every sequence were written"
            else:
                batch = rng.choice([1, 2, 7, 16, 33])
                maxl = rng.choice([1, 2, 63, 64, 65, 300, 1300, 4200])
                minl = rng.choice([1, 1, maxl])
                w = pkg.workloads.paged_decode(seed=seed * 31 + case, batch=batch, heads=kvh, head_dim=d, min_len=minl, max_len=maxl,
                                               pool_slots=max(2048, batch * (maxl + 2)), dtype=dtype, index_dtype=idt)
                desc += f" batch={batch} len {minl}..{maxl}"
                q = torch.randn(batch, heads, d, generator=g).to(dtype)
                kp, vp = w["k_pool"], w["v_pool"]
                want = oracle.token_attention(q.float(), kp.float(), vp.float(), w["b_loc"], w["b_seq_len"], w["max_input_len"])
                args = (w["b_loc"].to(dev), w["b_start_loc"].to(dev), w["b_seq_len"].to(dev), w["max_input_len"])
                got = ops.token_decode_attention(q.to(dev), kp.to(dev), vp.to(dev), *args, no_alloc=(kind == "decode_noalloc"))
                (assert_fp32 if dtype == torch.float32 else assert_half)(got, want.to(dtype))
        except AssertionError as e:
            failed.append(desc + ": " + str(e)[:300])
        except RuntimeError as e:   # nothing in these ranges may be refused
            failed.append(desc + ": refused: " + str(e)[:300])
    _report(failed, n)


def _rand_shape(rng):
    nd = rng.choice([0, 1, 1, 2, 2, 3, 4])
    return tuple(rng.choice([1, 1, 2, 3, 5, 8, 17, 64, 100, 257]) for _ in range(nd))


def _broadcastable(rng, shape):
    s = list(shape)
    for i in range(len(s)):
        if rng.random() < 0.3:
            s[i] = 1
    drop = rng.randint(0, len(s))
    return tuple(s[drop:]) if rng.random() < 0.4 else tuple(s)


def _make(shape, dtype, g):
    if dtype.is_floating_point:
        return torch.randn(shape, generator=g).to(dtype)
    if dtype == torch.bool:
        return torch.rand(shape, generator=g) > 0.5
    return torch.randint(0 if dtype == torch.uint8 else -50, 50, shape, generator=g).to(dtype)


def _view_of(t, how, dev):
    """a non-contiguous device view with the values of t"""
    d = t.to(dev)
    if how == "t" and d.dim() >= 2:
        return d.transpose(-1, -2).contiguous().transpose(-1, -2)
    if how == "slice" and d.dim() >= 1 and d.shape[-1] >= 1:
        big = torch.zeros(*d.shape[:-1], d.shape[-1] * 2 + 1, dtype=d.dtype, device=dev)
        big[..., 1::2] = d
        return big[..., 1::2]
    return d


@pytest.mark.parametrize("seed,n", [(1, 500), (2, 500)])
def test_sweep_elementwise_and_rows(ops, dev, seed, n):
    """Binary ops with broadcasting, promotion, alpha, scalars, in-place forms and strided views; unary ops; comparisons;
    where; softmax over any dim; RMSNorm; mean; cat; copy with a dtype cast."""
    rng = random.Random(seed)
    rand_shape = lambda: _rand_shape(rng)
    broadcastable = lambda shape: _broadcastable(rng, shape)
    make = lambda shape, dtype, g, strided=False: _make(shape, dtype, g)
    view_of = lambda t, how: _view_of(t, how, dev)
    failed = []
    for case in range(n):
        g = torch.Generator().manual_seed(seed * 104729 + case)
        kind = rng.choice(["add", "sub", "mul", "div", "add_scalar", "mul_scalar", "silu", "unary", "softmax", "rms", "add_", "mul_", "cmp", "where", "mean", "cat", "copy"])
        desc = f"case {case} {kind}"
        try:
            if kind in ("add", "sub", "mul", "div", "add_", "mul_", "cmp", "where"):
                shape = rand_shape()
                da = rng.choice(FLOATS + INTS[:2])
                db = rng.choice(FLOATS + INTS[:2]) if rng.random() < 0.4 else da
                a = make(shape, da, g)
                b = make(broadcastable(shape), db, g)
                if kind in ("add_", "mul_"):
                    if torch.result_type(a, b) != a.dtype: b = b.to(a.dtype)
                va, vb = rng.choice(["c", "t", "slice"]), rng.choice(["c", "t", "slice"])
                alpha = rng.choice([1, 1, 2, -1, 0.5]) if kind in ("add", "sub", "add_") else 1
                if isinstance(alpha, float) and not torch.result_type(a, b).is_floating_point: alpha = 2
                desc += f" {da} {tuple(a.shape)}[{va}] {db} {tuple(b.shape)}[{vb}] alpha={alpha}"
                A, B = view_of(a, va), view_of(b, vb)
                if kind == "add":
                    want = torch.add(a, b, alpha=alpha)
                    got = ops.add(A, B, alpha=alpha)
                elif kind == "sub":
                    want = torch.sub(a, b, alpha=alpha)
                    got = ops.sub(A, B, alpha=alpha)
                elif kind == "mul":
                    want = torch.mul(a, b)
                    got = ops.mul(A, B)
                elif kind == "div":
                    if not b.dtype.is_floating_point:
                        b = b.masked_fill(b == 0, 3)
                        B = view_of(b, vb)
                    want = torch.div(a, b)
                    got = ops.div(A, B)
                elif kind == "add_":
                    want = a.clone().add_(b, alpha=alpha)
                    got = ops.add_(A, B, alpha=alpha)
                elif kind == "mul_":
                    want = a.clone().mul_(b)
                    got = ops.mul_(A, B)
                elif kind == "cmp":
                    op = rng.choice(["eq", "ne", "lt", "le", "gt", "ge"])
                    want = getattr(torch, op)(a, b)
                    got = getattr(ops, op)(A, B)
                else:
                    cond = make(shape, torch.bool, g)
                    if b.dtype != a.dtype:
                        b = b.to(a.dtype)
                        B = view_of(b, vb)
                    want = torch.where(cond, a, b)
                    got = ops.where(cond.to(dev), A, B)
                assert got.dtype == want.dtype, (got.dtype, want.dtype)
                assert_each(got, want)
            elif kind in ("add_scalar", "mul_scalar"):
                shape = rand_shape()
                da = rng.choice(FLOATS + INTS[:2])
                a = make(shape, da, g)
                sc = rng.choice([2, -3, 0.5, 1.25, 0])
                desc += f" {da} {shape} scalar={sc}"
                if kind == "add_scalar":
                    want = torch.add(a, sc)
                    got = ops.add(a.to(dev), sc)
                else:
                    want = torch.mul(a, sc)
                    got = ops.mul(a.to(dev), sc)
                assert got.dtype == want.dtype, (got.dtype, want.dtype)
                assert_each(got, want)
            elif kind in ("silu", "unary"):
                shape = rand_shape()
                da = rng.choice(FLOATS)
                a = make(shape, da, g)
                name = "silu" if kind == "silu" else rng.choice(["sigmoid", "neg", "sin", "cos", "exp", "rsqrt"])
                if name == "rsqrt": a = a.abs() + 0.1
                va = rng.choice(["c", "t", "slice"])
                desc += f" {name} {da} {shape}[{va}]"
                ref = {"silu": torch.nn.functional.silu, "sigmoid": torch.sigmoid, "neg": torch.neg, "sin": torch.sin, "cos": torch.cos, "exp": torch.exp, "rsqrt": torch.rsqrt}[name]
                want = ref(a.float()).to(da) if da == torch.float16 else ref(a)
                got = getattr(ops, name)(view_of(a, va))
                assert_each(got, want)
            elif kind == "softmax":
                shape = rand_shape() or (5,)
                da = rng.choice(FLOATS)
                a = make(shape, da, g)
                dim = rng.randrange(-len(shape), len(shape))
                desc += f" {da} {shape} dim={dim}"
                want = oracle.softmax(a, dim)
                got = ops.softmax(a.to(dev), dim)
                assert_close(got, want)
            elif kind == "rms":
                rows = rng.choice([1, 3, 64, 257])
                hdim = rng.choice([8, 64, 100, 512, 4096, 5000, 70000])
                da = rng.choice(FLOATS)
                a = make((rows, hdim), da, g)
                w = (torch.randn(hdim, generator=g) * 0.1 + 1).to(da)
                desc += f" {da} {(rows, hdim)}"
                want = oracle.rms_norm(a, w, 1e-5)
                got = ops.rms_norm(a.to(dev), w.to(dev), 1e-5)
                assert_close(got, want)
            elif kind == "mean":
                shape = rand_shape() or (7,)
                da = rng.choice(FLOATS)
                a = make(shape, da, g)
                dim = rng.randrange(-len(shape), len(shape))
                keep = rng.random() < 0.5
                desc += f" {da} {shape} dim={dim} keep={keep}"
                want = a.float().mean(dim, keepdim=keep).to(da)
                got = ops.mean(a.to(dev), [dim], keepdim=keep)
                assert_close(got, want)
            elif kind == "cat":
                shape = list(rand_shape() or (4,))
                dim = rng.randrange(len(shape))
                da = rng.choice(FLOATS + INTS[:2])
                parts = []
                for _ in range(rng.randint(1, 4)):
                    sh = list(shape)
                    sh[dim] = rng.choice([0, 1, 3, 17])
                    parts.append(make(tuple(sh), da, g))
                desc += f" {da} {[tuple(p.shape) for p in parts]} dim={dim}"
                want = torch.cat(parts, dim)
                got = ops.cat([p.to(dev) for p in parts], dim)
                assert_exact(got, want)
            else:
                shape = rand_shape()
                da = rng.choice(FLOATS + INTS)
                db = rng.choice(FLOATS + INTS)
                a = make(shape, da, g)
                if not db.is_floating_point and da.is_floating_point: a = (a * 10).round()
                if db == torch.uint8: a = a.abs()
                va = rng.choice(["c", "t", "slice"])
                desc += f" {da}->{db} {shape}[{va}]"
                dst = torch.zeros(shape, dtype=db, device=dev)
                ops.copy_(dst, view_of(a, va))
                want = a.to(db)
                assert_exact(dst, want)
        except AssertionError as e:
            failed.append(desc + ": " + str(e)[:300])
        except RuntimeError as e:   # nothing in these ranges may be refused
            failed.append(desc + ": refused: " + str(e)[:300])
    _report(failed, n)


@pytest.mark.parametrize("seed,n", [(1, 400), (2, 400)])
def test_sweep_rotary_index_and_batched(ops, dev, seed, n):
    """Rotary embedding (both pair conventions, table dtypes and widths), KV scatter, index_put, masked_fill, tril / triu,
    arange, index_select, gather, pow, bmm / baddbmm / matmul with transposed and broadcast operands, linear on 3-D
    input, and the projection with the rotary embedding in one call."""
    rng = random.Random(seed)
    failed = []
    for case in range(n):
        g = torch.Generator().manual_seed(seed * 15485863 + case)
        kind = rng.choice(["rotary", "rotary", "scatter", "index_put", "masked_fill", "tri", "arange", "index_select", "gather", "pow", "bmm", "matmul", "baddbmm", "linear3d", "linear_rotary"])
        desc = f"case {case} {kind}"
        try:
            if kind == "rotary":
                dt = rng.choice(FLOATS)
                tdt = rng.choice([dt, torch.float32])
                toks, heads, d = rng.choice([1, 5, 64, 300]), rng.choice([1, 3, 8, 32]), rng.choice([8, 32, 64, 80, 128, 256])
                inter, conj = rng.random() < 0.5, rng.random() < 0.3
                full = rng.random() < 0.3 and not inter   # half-split accepts full-width tables
                desc += f" {dt} table {tdt} [{toks},{heads},{d}] interleaved={inter} conj={conj} fullwidth={full}"
                x = torch.randn(toks, heads, d, generator=g).to(dt)
                cos, sin = oracle.precompute_freqs(d, toks)
                cos, sin = cos.to(tdt), sin.to(tdt)
                sgn = -1.0 if conj else 1.0
                want = (oracle.rotary_emb_interleaved if inter else oracle.rotary_emb)(x, cos.float(), sgn * sin.float())
                ct, st = (torch.cat([cos, cos], -1), torch.cat([sin, sin], -1)) if full else (cos, sin)
                got = ops.rotary_emb(x.to(dev), ct.to(dev), st.to(dev), conj=conj, interleaved=inter)
                assert_close(got, want.to(dt))
            elif kind == "scatter":
                dt = rng.choice(FLOATS + [torch.int8])
                idt = rng.choice([torch.int32, torch.int64])
                toks, heads, d, slots = rng.choice([1, 7, 64, 200]), rng.choice([1, 4, 32]), rng.choice([16, 64, 80, 128]), rng.choice([256, 1000])
                desc += f" {dt} idx {idt} [{toks},{heads},{d}] -> {slots}"
                k = (torch.randn(toks, heads, d, generator=g) * 20).to(dt)
                pool = (torch.randn(slots, heads, d, generator=g) * 20).to(dt)
                loc = torch.randperm(slots, generator=g)[:toks].to(idt)
                want = oracle.dest_index_copy_kv(pool.clone(), k, loc)
                dp = pool.to(dev)
                ops.dest_index_copy_kv(k.to(dev), loc.to(dev), dp)
                assert_exact(dp, want)
            elif kind == "index_put":
                dt = rng.choice(FLOATS + [torch.int64])
                rows, cols = rng.choice([4, 33, 500]), rng.choice([1, 8, 100])
                cnt = rng.choice([1, 3, rows])
                acc = rng.random() < 0.4
                desc += f" {dt} [{rows},{cols}] n={cnt} accumulate={acc}"
                x = (torch.randn(rows, cols, generator=g) * 10).to(dt)
                v = (torch.randn(cnt, cols, generator=g) * 10).to(dt)
                idx = torch.randperm(rows, generator=g)[:cnt]
                want = x.clone().index_put_((idx,), v, accumulate=acc)
                dx = x.to(dev)
                ops.index_put_(dx, (idx.to(dev),), v.to(dev), accumulate=acc)
                (assert_exact if not acc or not dt.is_floating_point else assert_close)(dx, want)
            elif kind == "masked_fill":
                dt = rng.choice(FLOATS + [torch.int32])
                shape = (rng.choice([1, 3, 17]), rng.choice([1, 8, 130]))
                mshape = rng.choice([shape, (1, shape[1]), (shape[0], 1), (shape[1],)])
                val = rng.choice([0, -1, 2.5, float("-inf")]) if dt.is_floating_point else rng.choice([0, 7])
                desc += f" {dt} {shape} mask {mshape} value={val}"
                x = (torch.randn(shape, generator=g) * 5).to(dt)
                m = torch.rand(mshape, generator=g) > 0.5
                want = x.masked_fill(m, val)
                got = ops.masked_fill(x.to(dev), m.to(dev), val)
                assert_exact(got, want)
            elif kind == "tri":
                dt = rng.choice(FLOATS + [torch.int64, torch.bool])
                shape = rng.choice([(5, 5), (3, 7), (2, 9, 4), (1, 1), (130, 70)])
                diag = rng.choice([0, 0, 1, -1, 3, -10, 100])
                up = rng.random() < 0.5
                desc += f" {'triu' if up else 'tril'} {dt} {shape} diag={diag}"
                x = (torch.randn(shape, generator=g) * 5).to(dt) if dt != torch.bool else torch.rand(shape, generator=g) > 0.3
                want = (torch.triu if up else torch.tril)(x, diag)
                got = (ops.triu if up else ops.tril)(x.to(dev), diag)
                assert_exact(got, want)
            elif kind == "arange":
                dt = rng.choice([torch.int64, torch.int32, torch.float32, torch.bfloat16, torch.float16])
                start, step = rng.choice([0, 3, -5]), rng.choice([1, 2, 3, -1])
                cnt = rng.choice([0, 1, 7, 128, 1000])
                if dt in (torch.bfloat16, torch.float16): cnt = min(cnt, 80)   # every value exactly representable
                end = start + step * cnt
                desc += f" {dt} {start}:{end}:{step}"
                want = torch.arange(start, end, step, dtype=dt)
                got = ops.arange(start, end, step, dtype=dt, device=dev)
                assert_exact(got, want)
            elif kind == "index_select":
                dt = rng.choice(FLOATS + [torch.int64])
                shape = (rng.choice([1, 6, 40]), rng.choice([1, 9, 64]), rng.choice([1, 5]))
                dim = rng.randrange(-3, 3)
                cnt = rng.choice([0, 1, 5, 100])
                idt = rng.choice([torch.int32, torch.int64])
                desc += f" {dt} {shape} dim={dim} n={cnt} {idt}"
                x = (torch.randn(shape, generator=g) * 5).to(dt)
                idx = torch.randint(0, shape[dim], (cnt,), generator=g).to(idt)
                want = x.index_select(dim, idx.long())
                got = ops.index_select(x.to(dev), dim, idx.to(dev))
                assert_exact(got, want)
            elif kind == "gather":
                dt = rng.choice(FLOATS + [torch.int32])
                shape = (rng.choice([1, 6, 40]), rng.choice([1, 9, 64]))
                dim = rng.randrange(-2, 2)
                ishape = (rng.randint(1, shape[0]), rng.randint(1, shape[1]))
                desc += f" {dt} {shape} dim={dim} index {ishape}"
                x = (torch.randn(shape, generator=g) * 5).to(dt)
                idx = torch.randint(0, shape[dim], ishape, generator=g)
                want = x.gather(dim, idx)
                got = ops.gather(x.to(dev), dim, idx.to(dev))
                assert_exact(got, want)
            elif kind == "pow":
                dt = rng.choice(FLOATS)
                shape = (rng.choice([1, 7, 300]), rng.choice([1, 64]))
                ex = rng.choice([2, 2.0, 0.5, -0.5, 3, -1, 0])
                desc += f" {dt} {shape} exponent={ex}"
                x = torch.rand(shape, generator=g).to(dt) + 0.25
                want = torch.pow(x.float(), ex).to(dt) if dt == torch.float16 else torch.pow(x, ex)
                got = ops.pow(x.to(dev), ex)
                assert_each(got, want)
            elif kind in ("bmm", "baddbmm"):
                dt = rng.choice(FLOATS)
                bt, m, k, nn = rng.choice([1, 3, 16]), rng.choice([1, 17, 128, 300]), rng.choice([8, 64, 136, 512]), rng.choice([8, 40, 256, 1000])
                ta, tb = rng.random() < 0.4, rng.random() < 0.4
                desc += f" {dt} b={bt} m={m} k={k} n={nn} transA={ta} transB={tb}"
                a = torch.randn(bt, m, k, generator=g).to(dt)
                b = (torch.randn(bt, k, nn, generator=g) * 0.1).to(dt)
                A = a.to(dev).transpose(1, 2).contiguous().transpose(1, 2) if ta else a.to(dev)
                B = b.to(dev).transpose(1, 2).contiguous().transpose(1, 2) if tb else b.to(dev)
                want = torch.bmm(a.float(), b.float())
                if kind == "bmm":
                    got = ops.bmm(A, B)
                else:
                    c = torch.randn(rng.choice([(bt, m, nn), (1, m, nn), (bt, 1, nn)]), generator=g).to(dt)
                    beta, alpha = rng.choice([1, 0.5, 0]), rng.choice([1, 2])
                    want = beta * c.float() + alpha * want if beta != 0 else alpha * want
                    got = ops.baddbmm(c.to(dev), A, B, beta=beta, alpha=alpha)
                (assert_fp32 if dt == torch.float32 else assert_half)(got, want, **({} if dt == torch.float32 else {"abs_": 1e-2 * max(1.0, float(want.abs().max()) / 8)}))
            elif kind == "matmul":
                dt = rng.choice(FLOATS)
                form = rng.choice(["vv", "mv", "vm", "bm_m", "m_bm", "bb", "bcast"])
                k = rng.choice([8, 64, 136])
                sh = {"vv": ((k,), (k,)), "mv": ((17, k), (k,)), "vm": ((k,), (k, 33)), "bm_m": ((3, 17, k), (k, 40)), "m_bm": ((17, k), (4, k, 24)),
                      "bb": ((2, 3, 9, k), (2, 3, k, 16)), "bcast": ((2, 1, 9, k), (3, k, 16))}[form]
                desc += f" {dt} {sh}"
                a = torch.randn(sh[0], generator=g).to(dt)
                b = (torch.randn(sh[1], generator=g) * 0.1).to(dt)
                want = torch.matmul(a.float(), b.float())
                got = ops.matmul(a.to(dev), b.to(dev))
                (assert_fp32 if dt == torch.float32 else assert_half)(got, want)
            elif kind == "linear3d":
                dt = rng.choice(FLOATS)
                b0, s0, k, nn = rng.choice([1, 2, 5]), rng.choice([1, 7, 129]), rng.choice([64, 256, 1000]), rng.choice([8, 136, 4096])
                bias = rng.random() < 0.5
                desc += f" {dt} [{b0},{s0},{k}] -> {nn} bias={bias}"
                x = torch.randn(b0, s0, k, generator=g).to(dt)
                w = (torch.randn(nn, k, generator=g) * 0.05).to(dt)
                bb = torch.randn(nn, generator=g).to(dt) if bias else None
                want = torch.nn.functional.linear(x.float(), w.float(), bb.float() if bias else None)
                got = ops.linear(x.to(dev), w.to(dev), bb.to(dev) if bias else None)
                (assert_fp32 if dt == torch.float32 else assert_half)(got, want)
            else:
                dt = rng.choice([torch.bfloat16, torch.float16])
                tdt = rng.choice([dt, torch.float32])
                m, heads, hd, vcols, k = rng.choice([1, 9, 64, 300, 1100]), rng.choice([1, 4, 24, 96]), rng.choice([64, 128]), rng.choice([0, 64, 1024]), rng.choice([64, 128, 384])
                inter, conj, bias = rng.random() < 0.7, rng.random() < 0.3, rng.random() < 0.4
                desc += f" {dt} table {tdt} m={m} heads={heads}x{hd} +{vcols} k={k} interleaved={inter} conj={conj} bias={bias}"
                rot = heads * hd
                nn = rot + vcols
                x = torch.randn(m, k, generator=g).to(dt)
                w = (torch.randn(nn, k, generator=g) * 0.05).to(dt)
                bb = torch.randn(nn, generator=g).to(dt) if bias else None
                cos, sin = oracle.precompute_freqs(hd, m)
                cos, sin = cos.to(tdt), sin.to(tdt)
                y = x.float() @ w.float().t() + (bb.float() if bias else 0)
                sgn = -1.0 if conj else 1.0
                wr = (oracle.rotary_emb_interleaved if inter else oracle.rotary_emb)(y[:, :rot].reshape(m, heads, hd), cos.float(), sgn * sin.float())
                want = torch.cat([wr.reshape(m, rot), y[:, rot:]], 1)
                got = ops.linear_rotary(x.to(dev), w.to(dev), cos.to(dev), sin.to(dev), rot, hd, bb.to(dev) if bias else None, conj=conj, interleaved=inter)
                # where the projection and the rotation run as two ops the projection is rounded to the output dtype in
                # between, as the reference's two calls do: up to one 16-bit ulp of a value of magnitude 4
                assert_half(got, want, abs_=3e-2)
        except AssertionError as e:
            failed.append(desc + ": " + str(e)[:300])
        except RuntimeError as e:   # nothing in these ranges may be refused
            failed.append(desc + ": refused: " + str(e)[:300])
    _report(failed, n)


@pytest.mark.parametrize("seed,n", [(1, 400), (2, 400)])
def test_sweep_strided_operands_and_argument_forms(ops, dev, pkg, seed, n):
    """q / k / v as views of one packed projection and a strided destination for prefill attention, K and V as the halves
    of one packed pool for decode, RMSNorm with bias / inv_rms on n-d input, rotary in place on a packed view, softmax on
    transposed input, div rounding modes, comparisons with scalars, masked_fill with a value tensor, fill on hollow views,
    broadcast copies with a cast into a transposed destination, in-place ops on hollow views."""
    rng = random.Random(seed)
    failed = []
    for case in range(n):
        g = torch.Generator().manual_seed(seed * 32452843 + case)
        kind = rng.choice(["prefill_packed", "decode_strided", "rms_forms", "rotary_strided", "softmax_strided", "div_modes", "cmp_scalar", "masked_fill_tensor", "fill", "copy_bcast", "silu_mul", "sub_scalar", "linear_out_strided3d", "where_scalar", "inplace_strided"])
        desc = f"case {case} {kind}"
        try:
            if kind == "prefill_packed":
                dt = rng.choice(FLOATS)
                d = rng.choice([64, 128, 80])
                kvh = rng.choice([1, 2, 4])
                heads = kvh * rng.choice([1, 2, 4])
                lens = [rng.randint(1, 300 if dt != torch.float32 and d != 80 else 150) for _ in range(rng.choice([1, 2, 4]))]
                toks = sum(lens)
                starts = [sum(lens[:i]) for i in range(len(lens))]
                desc += f" {dt} heads={heads}/{kvh} d={d} lens={lens}"
                qkv = torch.randn(toks, (heads + 2 * kvh) * d, generator=g).to(dt)
                q, k, v = qkv[:, :heads * d].view(toks, heads, d), qkv[:, heads * d:(heads + kvh) * d].view(toks, kvh, d), qkv[:, (heads + kvh) * d:].view(toks, kvh, d)
                st, ln = torch.tensor(starts, dtype=torch.int32), torch.tensor(lens, dtype=torch.int32)
                want = oracle.context_attention(q.contiguous(), k.contiguous(), v.contiguous(), st, ln)
                dq = qkv.to(dev)
                Q, K, V = dq[:, :heads * d].view(toks, heads, d), dq[:, heads * d:(heads + kvh) * d].view(toks, kvh, d), dq[:, (heads + kvh) * d:].view(toks, kvh, d)
                big = torch.zeros(toks, heads * d + 16, dtype=dt, device=dev)
                out = big[:, :heads * d].view(toks, heads, d)
                ops.context_attention(Q, K, V, st.to(dev), ln.to(dev), max(lens), out=out)
                (assert_fp32 if dt == torch.float32 else assert_half)(out, want)
                assert float(big[:, heads * d:].abs().sum()) == 0.0
            elif kind == "decode_strided":
                dt = rng.choice(FLOATS)
                d = rng.choice([64, 128, 48])
                kvh = rng.choice([1, 2, 8])
                heads = kvh * rng.choice([1, 4])
                batch = rng.choice([1, 3, 9])
                maxl = rng.choice([1, 70, 600, 1100])
                desc += f" {dt} heads={heads}/{kvh} d={d} batch={batch} maxlen={maxl}"
                w = pkg.workloads.paged_decode(seed=seed * 13 + case, batch=batch, heads=kvh, head_dim=d, min_len=1, max_len=maxl, pool_slots=max(1024, batch * (maxl + 2)), dtype=dt)
                q = torch.randn(batch, heads, d, generator=g).to(dt)
                want = oracle.token_attention(q.float(), w["k_pool"].float(), w["v_pool"].float(), w["b_loc"], w["b_seq_len"], w["max_input_len"])
                # K and V as the two halves of one packed pool [slots, 2, kv_heads, d]; b_loc wider than max_input_len is not allowed, so keep it
                kv = torch.stack([w["k_pool"], w["v_pool"]], 1).to(dev)
                args = (w["b_loc"].to(dev), w["b_start_loc"].to(dev), w["b_seq_len"].to(dev), w["max_input_len"])
                qq = torch.zeros(batch, heads, d + 8, dtype=dt, device=dev)
                qq[..., :d] = q.to(dev)
                got = ops.token_decode_attention(qq[..., :d] if d % 8 == 0 else q.to(dev), kv[:, 0], kv[:, 1], *args)
                (assert_fp32 if dt == torch.float32 else assert_half)(got, want.to(dt))
            elif kind == "rms_forms":
                dt = rng.choice(FLOATS)
                shape = rng.choice([(3, 5, 64), (2, 2, 2, 100), (7, 4096), (1, 8), (300, 1000)])
                bias = rng.random() < 0.4
                inv = rng.random() < 0.5
                desc += f" {dt} {shape} bias={bias} inv_rms={inv}"
                x = torch.randn(shape, generator=g).to(dt)
                wt = (torch.randn(shape[-1], generator=g) * 0.1 + 1).to(dt)
                b = torch.randn(shape[-1], generator=g).to(dt) if bias else None
                want = oracle.rms_norm(x, wt, 1e-6)
                if bias:   # one rounding, after the bias: the norm in fp32 (rms_norm_fp32 follows model.py:34-39)
                    xf = x.float()
                    want = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6) * wt.float() + b.float()).to(dt)
                ir = torch.empty(shape[:-1], dtype=torch.float32, device=dev) if inv else None
                got = ops.rms_norm(x.to(dev), wt.to(dev), 1e-6, bias=b.to(dev) if bias else None, inv_rms=ir)
                assert_close(got, want)
                if inv: assert_fp32(ir, torch.rsqrt(x.float().pow(2).mean(-1) + 1e-6), rel=1e-5)
            elif kind == "rotary_strided":
                dt = rng.choice(FLOATS)
                toks, heads, d = rng.choice([1, 33, 200]), rng.choice([2, 8]), rng.choice([64, 128, 32])
                inter = rng.random() < 0.5
                desc += f" {dt} [{toks},{heads},{d}] interleaved={inter} packed qkv view, in place"
                qkv = torch.randn(toks, 3 * heads * d, generator=g).to(dt)
                cos, sin = oracle.precompute_freqs(d, toks)
                cos, sin = cos.to(dt), sin.to(dt)
                want = qkv.clone()
                wq = (oracle.rotary_emb_interleaved if inter else oracle.rotary_emb)(qkv[:, :heads * d].reshape(toks, heads, d), cos.float(), sin.float())
                want[:, :heads * d] = wq.reshape(toks, heads * d).to(dt)
                dq = qkv.to(dev)
                view = dq[:, :heads * d].view(toks, heads, d)
                ops.rotary_emb(view, cos.to(dev), sin.to(dev), interleaved=inter, out=view)
                assert_close(dq[:, :heads * d], want[:, :heads * d])
                assert_exact(dq[:, heads * d:], want[:, heads * d:])
            elif kind == "softmax_strided":
                dt = rng.choice(FLOATS)
                shape = rng.choice([(4, 8, 33), (2, 3, 5, 7), (64, 300), (5, 70000)])
                dim = rng.randrange(-len(shape), len(shape))
                desc += f" {dt} {shape} dim={dim} transposed input"
                x = torch.randn(shape, generator=g).to(dt)
                X = x.to(dev).transpose(0, -1).contiguous().transpose(0, -1)
                assert_close(ops.softmax(X, dim), oracle.softmax(x, dim))
            elif kind == "div_modes":
                dt = rng.choice(FLOATS + [torch.int32, torch.int64])
                mode = rng.choice([None, "floor", "trunc"])
                shape = rng.choice([(7,), (3, 50), (2, 1, 9)])
                desc += f" {dt} {shape} mode={mode}"
                a = (torch.randn(shape, generator=g) * 20).to(dt)
                b = (torch.randn(shape[-1:], generator=g) * 5).to(dt)
                b = torch.where(b == 0, torch.ones_like(b) * 3, b)
                if dt.is_floating_point and mode is not None: a, b = a.round(), b.round().masked_fill(b.round() == 0, 2)
                want = torch.div(a.float(), b.float(), rounding_mode=mode).to(dt) if dt == torch.float16 else torch.div(a, b, rounding_mode=mode)
                got = ops.div(a.to(dev), b.to(dev), rounding_mode=mode)
                assert got.dtype == want.dtype, (got.dtype, want.dtype)
                assert_each(got, want)
            elif kind == "cmp_scalar":
                dt = rng.choice(FLOATS + [torch.int32])
                op = rng.choice(["eq", "ne", "lt", "le", "gt", "ge"])
                sc = rng.choice([0, 1, -2, 0.5])
                desc += f" {op} {dt} scalar={sc}"
                a = torch.randint(-3, 4, (5, 40), generator=g).to(dt)
                assert_exact(getattr(ops, op)(a.to(dev), sc), getattr(torch, op)(a, sc))
            elif kind == "masked_fill_tensor":
                dt = rng.choice(FLOATS + [torch.int64])
                shape = (rng.choice([1, 6]), rng.choice([1, 33]))
                desc += f" {dt} {shape} value tensor (cpu / device), in place"
                x = (torch.randn(shape, generator=g) * 5).to(dt)
                m = torch.rand(shape, generator=g) > 0.5
                val = torch.tensor(3, dtype=dt)
                want = x.masked_fill(m, val)
                dx = x.to(dev)
                ops.masked_fill_(dx, m.to(dev), val if rng.random() < 0.5 else val.to(dev))
                assert_exact(dx, want)
            elif kind == "fill":
                dt = rng.choice(FLOATS + [torch.int32, torch.int64, torch.bool, torch.uint8])
                shape = rng.choice([(), (1,), (1000,), (3, 4, 5)])
                v = rng.choice([0, 1, 7]) if not dt.is_floating_point else rng.choice([0.0, -2.5, 1e4])
                if dt == torch.bool: v = bool(v)
                desc += f" {dt} {shape} value={v}"
                x = torch.zeros(shape, dtype=dt, device=dev)
                big = torch.zeros((6, 10), dtype=dt, device=dev)
                ops.fill_(x, v)
                ops.fill_(big[::2, 1::3], v)
                assert_exact(x, torch.full(shape, v, dtype=dt))
                wb = torch.zeros((6, 10), dtype=dt)
                wb[::2, 1::3] = v
                assert_exact(big, wb)
            elif kind == "copy_bcast":
                da, db = rng.choice(FLOATS + [torch.int32]), rng.choice(FLOATS + [torch.int64])
                desc += f" {da}->{db} broadcast + transposed destination"
                src = torch.randint(-20, 20, (1, 7), generator=g).to(da)
                dst = torch.zeros(7, 5, dtype=db, device=dev).t()
                ops.copy_(dst, src.to(dev).expand(5, 7))
                assert_exact(dst.contiguous(), src.to(db).expand(5, 7).contiguous())
            elif kind == "silu_mul":
                dt = rng.choice(FLOATS)
                shape = rng.choice([(1, 8), (33, 1000), (4, 3, 64)])
                desc += f" {dt} {shape}"
                a, b = torch.randn(shape, generator=g).to(dt), torch.randn(shape, generator=g).to(dt)
                want = (torch.nn.functional.silu(a.float()) * b.float()).to(dt)
                assert_close(ops.silu_mul(a.to(dev), b.to(dev)), want)
            elif kind == "sub_scalar":
                dt = rng.choice(FLOATS + [torch.int64])
                sc, al = rng.choice([1, 2.5, -3]), rng.choice([1, 2])
                if not dt.is_floating_point: sc = int(sc)
                desc += f" {dt} scalar={sc} alpha={al}"
                a = torch.randint(-9, 9, (4, 9), generator=g).to(dt)
                want = torch.sub(a, sc, alpha=al)
                got = ops.sub(a.to(dev), sc, alpha=al)
                assert got.dtype == want.dtype
                assert_each(got, want)
            elif kind == "linear_out_strided3d":
                dt = rng.choice(FLOATS)
                b0, s0, k, nn = rng.choice([1, 3]), rng.choice([1, 40]), rng.choice([64, 200]), rng.choice([8, 136])
                desc += f" {dt} [{b0},{s0},{k}] -> {nn} into a strided 3-D destination"
                x = torch.randn(b0, s0, k, generator=g).to(dt)
                wt = (torch.randn(nn, k, generator=g) * 0.1).to(dt)
                big = torch.zeros(b0, s0, nn + 8, dtype=dt, device=dev)
                ops.linear(x.to(dev), wt.to(dev), out=big[..., :nn])
                want = torch.nn.functional.linear(x.float(), wt.float())
                (assert_fp32 if dt == torch.float32 else assert_half)(big[..., :nn], want)
                assert float(big[..., nn:].abs().sum()) == 0
            elif kind == "where_scalar":
                dt = rng.choice(FLOATS + [torch.int64])
                shape = (rng.choice([1, 5]), rng.choice([1, 40]))
                desc += f" {dt} {shape}"
                c = torch.rand(shape, generator=g) > 0.5
                a = torch.randint(-5, 5, shape, generator=g).to(dt)
                assert_exact(ops.where(c.to(dev), a.to(dev), 0), torch.where(c, a, torch.zeros((), dtype=dt)))
                assert_exact(ops.where(c.to(dev), 1, a.to(dev)), torch.where(c, torch.ones((), dtype=dt), a))
            else:
                dt = rng.choice(FLOATS + [torch.int32])
                desc += f" {dt} add_/mul_ on a hollow view"
                base = torch.randint(-9, 9, (8, 12), generator=g).to(dt)
                other = torch.randint(-4, 4, (4, 4), generator=g).to(dt)
                want = base.clone()
                want[::2, 1:9:2] += 2 * other
                want[::2, 1:9:2] *= other
                db = base.to(dev)
                ops.add_(db[::2, 1:9:2], other.to(dev), alpha=2)
                ops.mul_(db[::2, 1:9:2], other.to(dev))
                assert_each(db, want)
        except AssertionError as e:
            failed.append(desc + ": " + str(e)[:300])
        except (RuntimeError, TypeError) as e:
            failed.append(desc + ": refused: " + type(e).__name__ + " " + str(e)[:300])
    _report(failed, n)
