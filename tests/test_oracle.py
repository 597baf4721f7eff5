"""Pins the CPU oracle (oracle/cpu_fallback.py) without a GPU: the reference's own
known-answer tests, float64 brute force on tiny inputs, library routines and invariants
chosen so that a dropped term, a wrong sign/index or a transposed operand fails."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import cpu_fallback as oracle


# ---- known answers held by the reference's tests --------------------------------------
def test_rsqrt_known_answer():
    # dipu/tests/python/unittests/test_rsqrt.py:8-15: gold = a ** -0.5
    x = torch.rand(10, generator=torch.Generator().manual_seed(666))
    gold = torch.tensor([float(a) ** -0.5 for a in x])
    assert torch.allclose(torch.rsqrt(x), gold, atol=1e-5)


def test_silu_known_answer():
    # test_silu.py:23-34: silu(1) in half vs float within 1e-2; value is 1/(1+e^-1)
    want = 1.0 / (1.0 + math.exp(-1.0))
    half = oracle.silu(torch.ones(2, dtype=torch.half))
    full = oracle.silu(torch.ones(2))
    assert abs(float(full[0]) - want) < 1e-6
    assert (half.float() - full).abs().max() < 1e-2
    assert half.dtype == torch.half


def test_linear_known_answer():
    # test_linear.py:14-46: weight = bias = 1, x = arange => y = sum(x_row) + 1
    for shape in [(3, 3), (2, 2, 3), (2, 2, 2, 3)]:
        x = torch.arange(math.prod(shape), dtype=torch.float).reshape(shape)
        y = oracle.linear(x, torch.ones(2, 3), torch.ones(2))
        want = x.sum(-1, keepdim=True).expand(*shape[:-1], 2) + 1
        assert torch.equal(y, want)


def test_index_put_known_answer():
    # test_index.py:78-86: x[arange(3)] = 1 fills everything, then = 0
    x = torch.randn(3, 4, 5)
    oracle.index_put_(x, [torch.arange(3)], torch.tensor(1.0))
    assert torch.equal(x, torch.ones(3, 4, 5))
    oracle.index_put_(x, [torch.arange(3)], torch.tensor(0.0))
    assert torch.equal(x, torch.zeros(3, 4, 5))


def test_fp16_is_computed_in_fp32_like_the_custom_fallback():
    # CustomFallbackFunctions.hpp:23-30: only fp16 is up-cast; bf16 stays bf16
    g = torch.Generator().manual_seed(0)
    a16 = torch.randn(8, 64, generator=g).half()
    b16 = torch.randn(64, 8, generator=g).half()
    assert torch.equal(oracle.mm(a16, b16), torch.mm(a16.float(), b16.float()).half())
    abf = a16.bfloat16()
    assert oracle.softmax(abf, -1).dtype == torch.bfloat16
    assert torch.equal(oracle.softmax(abf, -1), torch.softmax(abf, -1))


# ---- RMSNorm ------------------------------------------------------------------------------
def test_rms_norm_brute_force_and_library():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 24, generator=g, dtype=torch.float64)
    w = torch.randn(24, generator=g, dtype=torch.float64)
    eps = 1e-6
    got = oracle.rms_norm(x, w, eps)
    want = np.empty((5, 24))
    xn, wn = x.numpy(), w.numpy()
    for r in range(5):
        ms = sum(float(v) ** 2 for v in xn[r]) / 24
        for c in range(24):
            want[r, c] = xn[r, c] / math.sqrt(ms + eps) * wn[c]
    assert np.allclose(got.numpy(), want, rtol=1e-12, atol=1e-12)
    assert torch.allclose(got, F.rms_norm(x, (24,), w, eps), rtol=1e-12, atol=1e-12)
    # scale invariance for eps -> 0, and the fp32-internal variant agrees in fp32
    assert torch.allclose(oracle.rms_norm(3.0 * x, w, 0.0), oracle.rms_norm(x, w, 0.0), rtol=1e-12)
    xf = x.float()
    assert torch.allclose(oracle.rms_norm_fp32(xf, w.float(), eps), oracle.rms_norm(xf, w.float(), eps), rtol=1e-5, atol=1e-6)


# ---- rotary -------------------------------------------------------------------------------
def test_rotary_invariants():
    g = torch.Generator().manual_seed(2)
    seq, heads, d = 16, 3, 8
    x = torch.randn(seq, heads, d, generator=g, dtype=torch.float64)
    cos, sin = oracle.precompute_freqs(d, seq)
    cos, sin = cos.double(), sin.double()
    y = oracle.rotary_emb(x, cos, sin)
    # position 0 is the identity
    assert torch.allclose(y[0], x[0], atol=1e-12)
    # each (i, i + d/2) pair keeps its norm
    n_in = x[..., : d // 2] ** 2 + x[..., d // 2:] ** 2
    n_out = y[..., : d // 2] ** 2 + y[..., d // 2:] ** 2
    assert torch.allclose(n_in, n_out, atol=1e-6)
    # explicit element: o0 = x0 cos - x1 sin, o1 = x0 sin + x1 cos
    t, h, i = 5, 1, 2
    c, s = float(cos[t, i]), float(sin[t, i])
    assert abs(float(y[t, h, i]) - (float(x[t, h, i]) * c - float(x[t, h, i + d // 2]) * s)) < 1e-12
    assert abs(float(y[t, h, i + d // 2]) - (float(x[t, h, i]) * s + float(x[t, h, i + d // 2]) * c)) < 1e-12
    # R(p) R(q) = R(p + q): rotate everything by position 3 then 4 == by 7
    c3, s3 = cos[3:4].expand(seq, -1), sin[3:4].expand(seq, -1)
    c4, s4 = cos[4:5].expand(seq, -1), sin[4:5].expand(seq, -1)
    c7, s7 = cos[7:8].expand(seq, -1), sin[7:8].expand(seq, -1)
    assert torch.allclose(oracle.rotary_emb(oracle.rotary_emb(x, c3, s3), c4, s4), oracle.rotary_emb(x, c7, s7), atol=1e-6)


def test_precompute_freqs_closed_form():
    # dicp/test/model/llama/model.py:42-47: angle[t, i] = t * theta ** (-2 i / dim), evaluated here in
    # Python float arithmetic, element by element, for two bases and two head dims.
    for dim, end, theta in [(8, 9, 10000.0), (16, 33, 10000.0), (12, 7, 500.0), (128, 5, 10000.0)]:
        cos, sin = oracle.precompute_freqs(dim, end, theta)
        assert cos.shape == (end, dim // 2) and sin.shape == (end, dim // 2)
        for t in range(end):
            for i in range(dim // 2):
                ang = t * theta ** (-2.0 * i / dim)
                assert abs(float(cos[t, i]) - math.cos(ang)) < 2e-6, (dim, t, i)
                assert abs(float(sin[t, i]) - math.sin(ang)) < 2e-6, (dim, t, i)
    # known values: pair 0 turns by one radian per position; the last pair of a 128-wide head by 10000^(-126/128)
    cos, sin = oracle.precompute_freqs(128, 3)
    assert abs(float(cos[1, 0]) - 0.5403023058681398) < 1e-6 and abs(float(sin[2, 0]) - 0.9092974268256817) < 1e-6
    assert abs(float(sin[2, 63]) - math.sin(2 * 10000.0 ** (-126.0 / 128.0))) < 1e-9
    # the default base is 10000
    c2, s2 = oracle.precompute_freqs(128, 3, 10000.0)
    assert torch.equal(cos, c2) and torch.equal(sin, s2)


def test_rotary_half_split_equals_interleaved_under_permutation():
    g = torch.Generator().manual_seed(3)
    seq, heads, d = 12, 2, 16
    x = torch.randn(seq, heads, d, generator=g)
    cos, sin = oracle.precompute_freqs(d, seq)
    # interleaved layout of the same pairs: (x[i], x[i+d/2]) -> positions (2i, 2i+1)
    xi = torch.stack((x[..., : d // 2], x[..., d // 2:]), dim=-1).flatten(-2)
    yi = oracle.rotary_emb_interleaved(xi, cos, sin)
    y = oracle.rotary_emb(x, cos, sin)
    back = torch.cat((yi[..., 0::2], yi[..., 1::2]), dim=-1)
    assert torch.allclose(back, y, atol=1e-5)


# ---- KV scatter -----------------------------------------------------------------------------
def test_dest_index_copy_kv_brute_force():
    g = torch.Generator().manual_seed(4)
    pool = torch.randn(20, 2, 4, generator=g)
    before = pool.clone()
    k = torch.randn(5, 2, 4, generator=g)
    loc = torch.tensor([7, 0, 19, 3, 11], dtype=torch.int32)
    oracle.dest_index_copy_kv(pool, k, loc)
    for i in range(5):
        assert torch.equal(pool[int(loc[i])], k[i])
    untouched = [s for s in range(20) if s not in loc.tolist()]
    assert torch.equal(pool[untouched], before[untouched])


# ---- prefill attention ----------------------------------------------------------------------
def _brute_causal(q, k, v):
    n, heads, d = q.shape
    out = np.zeros((n, heads, d))
    qn, kn, vn = q.double().numpy(), k.double().numpy(), v.double().numpy()
    for h in range(heads):
        for i in range(n):
            sc = [float(np.dot(qn[i, h], kn[j, h])) / math.sqrt(d) for j in range(i + 1)]
            mx = max(sc)
            e = [math.exp(s - mx) for s in sc]
            z = sum(e)
            for j in range(i + 1):
                out[i, h] += e[j] / z * vn[j, h]
    return out


def test_context_attention_brute_force_library_and_invariants():
    g = torch.Generator().manual_seed(5)
    lens = [7, 1, 12]
    starts = [0, 7, 8]
    total, heads, d = 20, 2, 8
    q = torch.randn(total, heads, d, generator=g)
    k = torch.randn(total, heads, d, generator=g)
    v = torch.randn(total, heads, d, generator=g)
    out = oracle.context_attention(q, k, v, torch.tensor(starts), torch.tensor(lens))
    for s, n in zip(starts, lens):
        want = _brute_causal(q[s:s + n], k[s:s + n], v[s:s + n])
        assert np.allclose(out[s:s + n].numpy(), want, atol=1e-5)
        lib = F.scaled_dot_product_attention(q[s:s + n].transpose(0, 1), k[s:s + n].transpose(0, 1),
                                             v[s:s + n].transpose(0, 1), is_causal=True).transpose(0, 1)
        assert torch.allclose(out[s:s + n], lib, atol=1e-5)
        # the first query of every sequence sees only its own key: output = V[0]
        assert torch.allclose(out[s], v[s], atol=1e-6)
    # identical keys => uniform weights => running mean of V
    ku = k[:1].expand(total, -1, -1).contiguous()
    o2 = oracle.context_attention(q, ku, v, torch.tensor([0]), torch.tensor([total]))
    run_mean = torch.cumsum(v, 0) / torch.arange(1, total + 1).view(-1, 1, 1)
    assert torch.allclose(o2, run_mean, atol=1e-5)


def test_context_attention_grouped_kv_heads():
    g = torch.Generator().manual_seed(6)
    n, heads, kvh, d = 9, 4, 2, 8
    q = torch.randn(n, heads, d, generator=g)
    k = torch.randn(n, kvh, d, generator=g)
    v = torch.randn(n, kvh, d, generator=g)
    out = oracle.context_attention(q, k, v, torch.tensor([0]), torch.tensor([n]))
    want = _brute_causal(q, k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1))
    assert np.allclose(out.numpy(), want, atol=1e-5)


# ---- decode attention -----------------------------------------------------------------------
def test_token_attention_brute_force_and_len_one():
    g = torch.Generator().manual_seed(7)
    batch, heads, d, slots = 3, 2, 8, 40
    lens = torch.tensor([5, 1, 9])
    max_len = 9
    perm = torch.randperm(slots, generator=g)
    b_loc = torch.zeros(batch, max_len, dtype=torch.int64)
    off = 0
    for b in range(batch):
        n = int(lens[b])
        b_loc[b, max_len - n:] = perm[off:off + n]
        off += n
    kp = torch.randn(slots, heads, d, generator=g)
    vp = torch.randn(slots, heads, d, generator=g)
    q = torch.randn(batch, heads, d, generator=g)
    out = oracle.token_attention(q, kp, vp, b_loc, lens, max_len)
    for b in range(batch):
        n = int(lens[b])
        sl = b_loc[b, max_len - n:].tolist()
        for h in range(heads):
            sc = [float(torch.dot(q[b, h].double(), kp[s, h].double())) / math.sqrt(d) for s in sl]
            mx = max(sc)
            e = [math.exp(x - mx) for x in sc]
            z = sum(e)
            want = sum((e[j] / z) * vp[sl[j], h].double() for j in range(n))
            assert torch.allclose(out[b, h].double(), want, atol=1e-5)
    # a sequence of length one returns its only value row
    assert torch.allclose(out[1], vp[int(b_loc[1, -1])], atol=1e-6)


def test_token_logits_brute_force_every_element_and_two_call_identity():
    # ext_ops.py:116-118 split in two calls: logits [heads, total] with sequence b's scores at columns
    # b_start_loc[b] .. +len_b, then softmax over that range times V. Grouped KV heads, starts that leave a gap.
    g = torch.Generator().manual_seed(17)
    batch, heads, kvh, d, slots = 3, 4, 2, 8, 64
    lens = torch.tensor([5, 1, 9])
    starts = torch.tensor([0, 6, 8])          # a one-column gap after sequence 0 and after sequence 1
    total = 17
    max_len = 11
    perm = torch.randperm(slots, generator=g)
    b_loc = torch.full((batch, max_len), -1, dtype=torch.int64)
    off = 0
    for b in range(batch):
        n = int(lens[b])
        b_loc[b, max_len - n:] = perm[off:off + n]
        off += n
    kp = torch.randn(slots, kvh, d, generator=g)
    vp = torch.randn(slots, kvh, d, generator=g)
    q = torch.randn(batch, heads, d, generator=g)
    att = oracle.token_logits(q, kp, b_loc, starts, lens, max_len, total)
    assert att.shape == (heads, total)
    want = np.zeros((heads, total))
    for b in range(batch):
        n, s = int(lens[b]), int(starts[b])
        sl = b_loc[b, max_len - n:].tolist()
        for h in range(heads):
            for j in range(n):
                acc = 0.0
                for t in range(d):
                    acc += float(q[b, h, t]) * float(kp[sl[j], h // (heads // kvh), t])
                want[h, s + j] = acc / math.sqrt(d)
    assert np.allclose(att.double().numpy(), want, atol=1e-5)
    assert float(att[:, 5].abs().max()) == 0.0 and float(att[:, 7].abs().max()) == 0.0
    # softmax over a sequence's own columns times its V rows is the fused definition's output
    fused = oracle.token_attention(q, kp, vp, b_loc, lens, max_len)
    for b in range(batch):
        n, s = int(lens[b]), int(starts[b])
        sl = b_loc[b, max_len - n:]
        v = vp[sl].repeat_interleave(heads // kvh, dim=1)            # n, heads, d
        p = att[:, s:s + n].softmax(-1)                              # heads, n
        assert torch.allclose(torch.einsum("hn,nhd->hd", p, v), fused[b], atol=1e-5)


# ---- int8 weight-only linear ----------------------------------------------------------------
def test_weight_only_int8_brute_force():
    g = torch.Generator().manual_seed(8)
    m, k, n = 3, 16, 5
    x = torch.randn(m, k, generator=g).bfloat16()
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    sc = (0.001 + 0.019 * torch.rand(n, generator=g)).half()
    out = oracle.weight_only_int8_linear(x, w, sc)
    for i in range(m):
        for j in range(n):
            want = sum(float(x[i, t]) * int(w[j, t]) for t in range(k)) * float(sc[j])
            assert abs(float(out[i, j]) - want) < 1e-4 * max(1.0, abs(want))


# ---- the decoder block composes the pieces ---------------------------------------------------
def test_decoder_block_matches_independent_composition():
    from __graft_entry__ import load_package
    wl = load_package().workloads
    x, p, cfg = wl.tiny_block(seed=0, batch=1, seq=16, hidden=64, heads=4, ffn=96)
    out, inter = oracle.decoder_block(x, p, cfg["heads"], cfg["eps"], cfg["theta"])
    # independent re-derivation with library routines
    h1 = F.rms_norm(x, (64,), p["norm1"], cfg["eps"])
    qkv = h1 @ p["wqkv"].t()
    q, k, v = [t.view(1, 16, 4, 16) for t in qkv.split(64, dim=-1)]
    cos, sin = oracle.precompute_freqs(16, 16)

    def rot(t):
        t0, t1 = t[..., :8], t[..., 8:]
        c, s = cos.view(1, 16, 1, 8), sin.view(1, 16, 1, 8)
        return torch.cat((t0 * c - t1 * s, t0 * s + t1 * c), -1)

    a = F.scaled_dot_product_attention(rot(q).transpose(1, 2), rot(k).transpose(1, 2), v.transpose(1, 2), is_causal=True)
    x1 = x + a.transpose(1, 2).reshape(1, 16, 64) @ p["wo"].t()
    h2 = F.rms_norm(x1, (64,), p["norm2"], cfg["eps"])
    want = x1 + (F.silu(h2 @ p["wgate"].t()) * (h2 @ p["wup"].t())) @ p["wdown"].t()
    assert torch.allclose(out, want, atol=1e-5)


# ---- selection / mask / gather helpers: known answers and brute force ---------------------------
def test_select_helpers_known_answers():
    # dipu/tests/python/unittests/test_gather.py:10-16
    t = torch.tensor([[1, 2], [3, 4]])
    assert oracle.gather(t, 1, torch.tensor([[0, 0], [1, 0]])).tolist() == [[1, 1], [4, 3]]
    # dipu/tests/python/unittests/test_arange.py:8-24
    assert oracle.arange(5, 20, 1).tolist() == list(range(5, 20))
    assert oracle.arange(10, -7, -3).tolist() == [10, 7, 4, 1, -2, -5]
    x = torch.arange(24.0).view(4, 6)
    for d in (-2, 0, 1):
        lo, up = oracle.tril(x, d), oracle.triu(x, d)
        for r in range(4):
            for c in range(6):
                assert lo[r, c] == (x[r, c] if c - r <= d else 0)
                assert up[r, c] == (x[r, c] if c - r >= d else 0)
    m = torch.tensor([[True, False], [False, True]])
    assert oracle.masked_fill(torch.ones(2, 2), m, 7).tolist() == [[7, 1], [1, 7]]
    assert oracle.where(m, torch.zeros(2, 2), torch.ones(2, 2)).tolist() == [[0, 1], [1, 0]]
    assert oracle.index_select(x, 1, torch.tensor([5, 0])).tolist() == [[5, 0], [11, 6], [17, 12], [23, 18]]
    assert oracle.compare("ge", torch.tensor([1, 2, 3]), 2).tolist() == [False, True, True]
