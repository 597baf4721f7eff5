"""GPU parity at the sizes the measured configurations state, where those sizes select kernel paths the small
cases do not reach: the persistent several-rows-per-wave row kernels (more than 4096 rows), decode attention with
more KV splits than one merge batch, the chunk growth beyond 64 x 512 tokens, and every op of the 7B-shaped layer
at batch 4 x seq 2048 fed with the oracle's own bf16 intermediates."""
import math

import pytest
import torch

from oracle import cpu_fallback as oracle
from tests.parity import assert_exact, assert_fp32, assert_half

pytestmark = pytest.mark.gpu


def g(seed):
    return torch.Generator().manual_seed(seed)


# ------------------------------------------------------------------ memory-bound ops, bf16 [8192, 4096]
@pytest.fixture(scope="module")
def c2(pkg):
    return pkg.workloads.memory_bound(seed=0)


def test_add_mul_at_8192x4096(ops, dev, c2):
    a, b = c2["a"], c2["b"]
    da, db = a.to(dev), b.to(dev)
    # one bf16 rounding of the exact sum / product on both sides: bit-identical
    assert_exact(ops.add(da, db), oracle.add(a, b))
    assert_exact(ops.mul(da, db), oracle.mul(a, b))
    assert_half(ops.add(da, db, alpha=-0.5), oracle.add(a.float(), b.float(), alpha=-0.5))
    y = da.clone()
    ops.add_(y, db)
    assert_exact(y, oracle.add(a, b))
    assert_half(ops.silu_mul(da, db), oracle.silu(a.float()) * b.float())


def test_softmax_at_8192x4096(ops, dev, c2):
    a = c2["a"]
    got = ops.softmax(a.to(dev), -1)
    assert_half(got, oracle.softmax(a.float(), -1))       # vs fp32 arithmetic
    assert_half(got, oracle.softmax(a, -1))               # vs the CPU fallback in bf16
    top = a[:64].float().argmax(-1, keepdim=True)
    assert torch.equal(got[:64].float().cpu().gather(-1, top).squeeze(-1), got[:64].float().cpu().max(-1).values)


def test_rms_norm_at_8192x4096(ops, dev, c2):
    a, w, eps = c2["a"], c2["rms_weight"], c2["eps"]
    inv = torch.empty(8192, dtype=torch.float32, device=dev)
    got = ops.rms_norm(a.to(dev), w.to(dev), eps, inv_rms=inv)
    assert_half(got, oracle.rms_norm(a.float(), w.float(), eps))
    assert_half(got, oracle.rms_norm(a, w, eps))
    assert_half(got, oracle.rms_norm_fp32(a, w, eps))
    assert_fp32(inv, torch.rsqrt(a.float().pow(2).mean(-1) + eps))
    # row counts around the switch from one row per wave to the persistent loop, and a ragged last round
    for rows in (4096, 4097, 8191, 12289):
        x = torch.randn(rows, 4096, generator=g(rows)).bfloat16()
        assert_half(ops.rms_norm(x.to(dev), w.to(dev), eps), oracle.rms_norm(x.float(), w.float(), eps))
        assert_half(ops.softmax(x.to(dev), -1), oracle.softmax(x.float(), -1))


def test_rotary_at_8192x32x128(ops, dev, c2):
    x, cos, sin = c2["rot_x"], c2["cos"], c2["sin"]
    want = oracle.rotary_emb(x.float(), cos.float(), sin.float())
    assert_half(ops.rotary_emb(x.to(dev), cos.to(dev), sin.to(dev)), want)
    wi = oracle.rotary_emb_interleaved(x.float(), cos.float(), sin.float())
    assert_half(ops.rotary_emb(x.to(dev), cos.to(dev), sin.to(dev), interleaved=True), wi)
    # the tables themselves: bf16 roundings of the closed form cos / sin(t * 10000^(-2 i / 128))
    for t, i in [(0, 0), (1, 0), (8191, 0), (4097, 17), (8191, 63)]:
        ang = t * 10000.0 ** (-2.0 * i / 128)
        assert abs(float(cos[t, i]) - math.cos(ang)) <= 2 ** -8 and abs(float(sin[t, i]) - math.sin(ang)) <= 2 ** -8


# ------------------------------------------------------------------ paged decode step, batch 64, lens 512..4096
def test_paged_decode_step_at_batch_64(ops, dev, pkg):
    w = pkg.workloads.paged_decode(seed=0)
    assert int(w["b_seq_len"].min()) >= 513 and int(w["b_seq_len"].max()) <= 4097 and w["max_input_len"] > 8 * 512
    dk, dv = w["k_pool"].to(dev), w["v_pool"].to(dev)
    ops.dest_index_copy_kv(w["k_new"].to(dev), w["dest_loc"].to(dev), dk)
    ops.dest_index_copy_kv(w["v_new"].to(dev), w["dest_loc"].to(dev), dv)
    kp, vp = w["k_pool"], w["v_pool"]          # updated in place on the host: the pool is 2 x 2 GiB
    oracle.dest_index_copy_kv(kp, w["k_new"], w["dest_loc"])
    oracle.dest_index_copy_kv(vp, w["v_new"], w["dest_loc"])
    for lo in range(0, kp.shape[0], 65536):    # bit-exact, written rows and every untouched slot
        assert torch.equal(dk[lo:lo + 65536].cpu(), kp[lo:lo + 65536])
        assert torch.equal(dv[lo:lo + 65536].cpu(), vp[lo:lo + 65536])
    want = oracle.token_attention(w["q"], kp, vp, w["b_loc"], w["b_seq_len"], w["max_input_len"])   # gathers per sequence, fp32 math
    args = (w["b_loc"].to(dev), w["b_start_loc"].to(dev), w["b_seq_len"].to(dev), w["max_input_len"])
    got = ops.token_decode_attention(w["q"].to(dev), dk, dv, *args)
    assert_half(got, want.float())
    att = torch.zeros(32, w["total_tokens"], dtype=torch.float32, device=dev)
    ops.token_attention(w["q"].to(dev), dk, att, *args)
    want_att = oracle.token_logits(w["q"], kp, w["b_loc"], w["b_start_loc"], w["b_seq_len"], w["max_input_len"], w["total_tokens"])
    assert_fp32(att, want_att, rel=1e-5)       # bf16 products are exact in fp32; only the summation order differs
    out2 = torch.empty_like(got)
    ops.token_softmax_reducev(att, dv, out2, *args)
    assert_half(out2, want.float())


@pytest.mark.parametrize("lens", [[32768, 700], [32769, 1], [40000, 33000, 5], [5000, 4097, 4096, 513]])
def test_token_attention_long_sequences(ops, dev, lens):
    """Few sequences, so the chunks are short: 256 splits of exactly 128 tokens, one token more (the chunk grows to 192),
    40 000 tokens (all three merged by the kernel for more than 64 splits), and 40 splits (five batches of the merge
    kernel for up to 64). Slots are drawn with repetition from a small pool."""
    heads, kvh, d, slots = 4, 2, 128, 8192
    batch, width = len(lens), max(lens)
    kp = torch.randn(slots, kvh, d, generator=g(50)).bfloat16()
    vp = torch.randn(slots, kvh, d, generator=g(51)).bfloat16()
    q = torch.randn(batch, heads, d, generator=g(52)).bfloat16()
    b_loc = torch.zeros(batch, width, dtype=torch.int32)
    for b, n in enumerate(lens):
        b_loc[b, width - n:] = torch.randint(0, slots, (n,), generator=g(53 + b), dtype=torch.int32)
    ln = torch.tensor(lens, dtype=torch.int32)
    st = torch.zeros(batch, dtype=torch.int32)
    st[1:] = torch.cumsum(ln, 0)[:-1]
    want = oracle.token_attention(q.float(), kp.float(), vp.float(), b_loc, ln, width)
    args = (b_loc.to(dev), st.to(dev), ln.to(dev), width)
    got = ops.token_decode_attention(q.to(dev), kp.to(dev), vp.to(dev), *args)
    assert_half(got, want)
    att = torch.zeros(heads, sum(lens), dtype=torch.float32, device=dev)
    ops.token_attention(q.to(dev), kp.to(dev), att, *args)
    assert_fp32(att, oracle.token_logits(q, kp, b_loc, st, ln, width, sum(lens)), rel=1e-5)
    out2 = torch.empty_like(got)
    ops.token_softmax_reducev(att, vp.to(dev), out2, *args)
    assert_half(out2, want)


@pytest.mark.parametrize("lens", [[2048], [9000, 8000, 77], [130] * 16])
def test_token_attention_few_sequences_at_32_heads(ops, dev, lens):
    """Small batches at the 7B head count: the chunk length follows the number of workgroups the chip needs (64-token
    chunks for one 2048-token sequence, 128-token chunks and 71 splits for the second case, and two chunks each, of
    128 and 2 tokens, for the third)."""
    heads, d, slots = 32, 128, 4096
    batch, width = len(lens), max(lens)
    kp = torch.randn(slots, heads, d, generator=g(70)).bfloat16()
    vp = torch.randn(slots, heads, d, generator=g(71)).bfloat16()
    q = torch.randn(batch, heads, d, generator=g(72)).bfloat16()
    b_loc = torch.zeros(batch, width, dtype=torch.int32)
    for b, n in enumerate(lens):
        b_loc[b, width - n:] = torch.randint(0, slots, (n,), generator=g(73 + b), dtype=torch.int32)
    ln = torch.tensor(lens, dtype=torch.int32)
    st = torch.zeros(batch, dtype=torch.int32)
    st[1:] = torch.cumsum(ln, 0)[:-1]
    want = oracle.token_attention(q.float(), kp.float(), vp.float(), b_loc, ln, width)
    got = ops.token_decode_attention(q.to(dev), kp.to(dev), vp.to(dev), b_loc.to(dev), st.to(dev), ln.to(dev), width)
    assert_half(got, want)


@pytest.mark.parametrize("score_dtype,idt", [(torch.float32, torch.int64), (torch.bfloat16, torch.int32)])
def test_token_attention_two_call_at_512_token_chunks(ops, dev, score_dtype, idt):
    """64 sequences of 2048..2600 tokens at 8 heads keep the 512-token chunks, whose scores and slot indices the two-call
    kernels stage per chunk. 64-bit and 32-bit tables, fp32 and 16-bit score tensors, and table entries that point
    outside the pool: their scores are -inf and they take no part in the softmax, as in the fused form."""
    heads, d, slots, batch = 8, 128, 16384, 64
    lens = torch.randint(2048, 2601, (batch,), generator=g(80))
    width, total = int(lens.max()), int(lens.sum())
    kp = torch.randn(slots, heads, d, generator=g(81)).bfloat16()
    vp = torch.randn(slots, heads, d, generator=g(82)).bfloat16()
    q = torch.randn(batch, heads, d, generator=g(83)).bfloat16()
    b_loc = torch.zeros(batch, width, dtype=idt)
    for b in range(batch):
        n = int(lens[b])
        b_loc[b, width - n:] = torch.randint(0, slots, (n,), generator=g(84 + b)).to(idt)
    ln = lens.to(idt)
    st = torch.zeros(batch, dtype=idt)
    st[1:] = torch.cumsum(ln, 0)[:-1]
    want_att = oracle.token_logits(q, kp, b_loc, st, ln, width, total)
    # entries outside the pool, in the first, a middle and the last chunk of a few sequences
    bad = [(0, 0, -1), (0, 700, slots), (3, 1500, slots + 12345), (17, int(lens[17]) - 1, -7), (63, 511, 1 << 30), (63, 512, -slots)]
    dead = torch.zeros(total, dtype=torch.bool)
    for b, t, val in bad:
        b_loc[b, width - int(lens[b]) + t] = val
        dead[int(st[b]) + t] = True
    want_att[:, dead] = float("-inf")
    args = (b_loc.to(dev), st.to(dev), ln.to(dev), width)
    att = torch.zeros(heads, total, dtype=score_dtype, device=dev)
    ops.token_attention(q.to(dev), kp.to(dev), att, *args)
    live = ~dead
    assert bool(torch.isneginf(att.cpu()[:, dead]).all())
    if score_dtype == torch.float32:
        assert_fp32(att.cpu()[:, live], want_att[:, live], rel=1e-5)
    else:
        assert_half(att.cpu()[:, live], want_att[:, live])
    # the second half from the scores the first half stored: softmax over each sequence's live tokens, times V
    stored = att.cpu().float()
    want = torch.zeros(batch, heads, d)
    for b in range(batch):
        n, s0 = int(lens[b]), int(st[b])
        sl = b_loc[b, width - n:].long().clamp(0, slots - 1)
        prob = torch.softmax(stored[:, s0:s0 + n], dim=-1)            # -inf scores weigh nothing
        want[b] = torch.einsum("hn,nhd->hd", prob, vp[sl].float())
    out = torch.empty(batch, heads, d, dtype=torch.bfloat16, device=dev)
    ops.token_softmax_reducev(att, vp.to(dev), out, *args)
    assert_half(out, want)
    fused = ops.token_decode_attention(q.to(dev), kp.to(dev), vp.to(dev), *args)
    assert_half(fused, want)


def test_token_attention_length_beyond_the_table_is_cut(ops, dev):
    """b_seq_len larger than max_input_len reads the table row's max_input_len columns and nothing before it."""
    heads, d, slots, width = 4, 128, 256, 600
    kp = torch.randn(slots, heads, d, generator=g(60)).bfloat16()
    vp = torch.randn(slots, heads, d, generator=g(61)).bfloat16()
    q = torch.randn(2, heads, d, generator=g(62)).bfloat16()
    b_loc = torch.randint(0, slots, (2, width), generator=g(63), dtype=torch.int32)
    st = torch.tensor([0, width], dtype=torch.int32)
    want = oracle.token_attention(q.float(), kp.float(), vp.float(), b_loc, torch.tensor([width, width]), width)
    over = torch.tensor([width + 77, 100000], dtype=torch.int32)
    got = ops.token_decode_attention(q.to(dev), kp.to(dev), vp.to(dev), b_loc.to(dev), st.to(dev), over.to(dev), width)
    assert_half(got, want)


# ------------------------------------------------------------------ the 7B-shaped layer, batch 4 x seq 2048, op by op
def test_llama7b_layer_every_op_at_full_size(ops, dev, pkg):
    """Each device op gets the oracle's bf16 intermediate as its input and is held to 2e-2 relative / 1e-2 absolute
    against the oracle's fp32 result of that one op, so rounding does not chain."""
    x, p, cfg = pkg.workloads.llama7b_layer(seed=0)
    b, s, hidden = x.shape
    heads, eps = cfg["heads"], cfg["eps"]
    hd, T, ffn = hidden // heads, b * s, p["wgate"].shape[0]
    bf = torch.bfloat16
    up = lambda t: t.to(dev)
    x2 = x.reshape(T, hidden)
    cos, sin = oracle.precompute_freqs(hd, s, cfg["theta"])
    cos, sin = cos.to(bf), sin.to(bf)

    # RMSNorm
    h1 = oracle.rms_norm(x2.float(), p["norm1"].float(), eps)
    assert_half(ops.rms_norm(up(x2), up(p["norm1"]), eps), h1)
    h1b = h1.to(bf)
    # stacked QKV projection, then the rotary embedding of q and k
    qkv = oracle.linear(h1b.float(), p["wqkv"].float())
    d_qkv = ops.linear(up(h1b), up(p["wqkv"]))
    assert_half(d_qkv, qkv)
    qkvb = qkv.to(bf)
    q32, k32, v32 = (t.reshape(b, s, heads, hd) for t in qkvb.float().split(hidden, dim=-1))
    rot = lambda t: torch.stack([oracle.rotary_emb(t[i], cos.float(), sin.float()) for i in range(b)])
    qr, kr = rot(q32), rot(k32)
    dq = up(qkvb).split(hidden, dim=-1)
    assert_half(ops.rotary_emb(dq[0].reshape(b, s, heads, hd), up(cos), up(sin)), qr)
    assert_half(ops.rotary_emb(dq[1].reshape(b, s, heads, hd), up(cos), up(sin)), kr)
    # the same two steps as one launch (rotation applied to the fp32 accumulators, adjacent-pair weight rows)
    w_perm = torch.cat([ops.interleave_rotary_rows(p["wqkv"][:hidden], hd), ops.interleave_rotary_rows(p["wqkv"][hidden:2 * hidden], hd),
                        p["wqkv"][2 * hidden:]], dim=0)
    fused = ops.linear_rotary(up(h1b), up(w_perm), up(cos), up(sin), 2 * hidden, hd, interleaved=True).cpu()
    fq, fk, fv = fused.split(hidden, dim=-1)
    unperm = lambda t: t.reshape(b, s, heads, hd // 2, 2).transpose(3, 4).reshape(b, s, heads, hd)
    q_acc, k_acc, v_acc = (t.reshape(b, s, heads, hd) for t in qkv.split(hidden, dim=-1))
    assert_half(unperm(fq), rot(q_acc))
    assert_half(unperm(fk), rot(k_acc))
    assert_half(fv.reshape(b, s, heads, hd), v_acc)
    del fused, fq, fk, fv, d_qkv
    # causal attention
    qrb, krb, vb = qr.to(bf).reshape(T, heads, hd), kr.to(bf).reshape(T, heads, hd), v32.to(bf).reshape(T, heads, hd)
    starts = torch.arange(b, dtype=torch.int32) * s
    lens = torch.full((b,), s, dtype=torch.int32)
    attn = oracle.context_attention(qrb.float(), krb.float(), vb.float(), starts, lens)
    assert_half(ops.context_attention(up(qrb), up(krb), up(vb), up(starts), up(lens), s), attn)
    attnb = attn.to(bf).reshape(T, hidden)
    # out projection + residual
    x1 = x2.float() + oracle.linear(attnb.float(), p["wo"].float())
    assert_half(ops.addmm(up(x2), up(attnb), up(p["wo"]).t()), x1)
    assert_half(ops.add(up(x2), ops.linear(up(attnb), up(p["wo"]))), x1)
    x1b = x1.to(bf)
    # RMSNorm
    h2 = oracle.rms_norm(x1b.float(), p["norm2"].float(), eps)
    assert_half(ops.rms_norm(up(x1b), up(p["norm2"]), eps), h2)
    h2b = h2.to(bf)
    # SiLU-gated projections
    gate = oracle.linear(h2b.float(), p["wgate"].float())
    upj = oracle.linear(h2b.float(), p["wup"].float())
    act = oracle.silu(gate) * upj
    assert_half(ops.linear_silu_mul(up(h2b), up(ops.interleave_gate_up(p["wgate"], p["wup"]))), act)
    d_gate = ops.linear(up(h2b), up(p["wgate"]))
    assert_half(d_gate, gate)
    assert_half(ops.silu_mul(up(gate.to(bf)), up(upj.to(bf))), oracle.silu(gate.to(bf).float()) * upj.to(bf).float())
    del d_gate, gate, upj
    actb = act.to(bf)
    # down projection + residual
    out = x1b.float() + oracle.linear(actb.float(), p["wdown"].float())
    assert_half(ops.addmm(up(x1b), up(actb), up(p["wdown"]).t()), out)
