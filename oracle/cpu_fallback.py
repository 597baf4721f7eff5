"""CPU oracle for the DIOPI transformer-inference path. TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module; nothing under deeplink.framework_amd/ does, and the product path never routes
through it.

What the reference executes when an op is not implemented on the device is stock ATen
CPU kernels: the generic boxed fallback
(dipu/torch_dipu/csrc_dipu/aten/RegisterDIPU.cpp:131-158) or the hand-written
custom_fallback_dipu_* functions, which move inputs to the CPU, up-cast fp16 (only fp16)
to fp32, call at::<op> and copy the result back
(dipu/torch_dipu/csrc_dipu/aten/ops/CustomFallbackFunctions.hpp:23-48,389-474).
So for the ops DIPU wraps, the oracle IS torch on CPU with that dtype rule.

The fused ops DIPU does not wrap (RMSNorm, rotary, KV scatter, prefill/decode attention)
are restated from the pure-PyTorch definitions the reference holds in
dicp/dicp/vendor/AscendGraph/ext_ops.py and dicp/test/model/llama/model.py; each function
cites the lines it follows. The int8 weight-only linear has no counterpart anywhere in
the reference; its definition is the closed form of the workload description.

Pinning (tests/test_oracle.py): reference known-answer tests
(dipu/tests/python/unittests/test_rsqrt.py:11, test_silu.py:31-34, test_linear.py:14-46,
test_index.py:78-104), float64 brute-force loops on tiny inputs, torch library routines
(F.rms_norm, F.scaled_dot_product_attention) and algebraic invariants (rotation composes
and preserves norms, position 0 is the identity, first causal row equals V[0], ...);
precompute_freqs by the closed form cos/sin(t * theta^(-2i/dim)) evaluated element by element for
two bases, token_logits by a float64 loop over every (sequence, head, token) with grouped KV heads
and gapped start columns, and by softmax(logits) @ V == token_attention.
Parity unpinned: the C signatures of the ext ops (nothing in the reference states them).
"""
import math

import torch
import torch.nn.functional as F


def _fallback_dtype(t):
    """CustomFallbackFunctions.hpp:23-30: fp16 is computed in fp32 on the CPU, bf16/fp32 natively."""
    return t.float() if t.dtype == torch.float16 else t


def _back(result, like):
    return result.to(like.dtype)


# ---- ops DIPU wraps: stock ATen CPU kernels ---------------------------------
def add(a, b, alpha=1):
    return torch.add(a, b, alpha=alpha)


def sub(a, b, alpha=1):
    return torch.sub(a, b, alpha=alpha)


def mul(a, b):
    return torch.mul(a, b)


def div(a, b, rounding_mode=None):
    return torch.div(a, b, rounding_mode=rounding_mode)


def silu(x):
    """custom_fallback_dipu_silu_out, CustomFallbackFunctions.hpp:32-48."""
    return _back(F.silu(_fallback_dtype(x)), x)


def softmax(x, dim):
    """custom_fallback_dipu__softmax_out, CustomFallbackFunctions.hpp:466-474."""
    return _back(torch.softmax(_fallback_dtype(x), dim), x)


def mm(a, b):
    """custom_fallback_dipu_mm_out, CustomFallbackFunctions.hpp:389-400."""
    return _back(torch.mm(_fallback_dtype(a), _fallback_dtype(b)), a)


def bmm(a, b):
    return _back(torch.bmm(_fallback_dtype(a), _fallback_dtype(b)), a)


def matmul(a, b):
    return _back(torch.matmul(_fallback_dtype(a), _fallback_dtype(b)), a)


def addmm(c, a, b, beta=1, alpha=1):
    return _back(torch.addmm(_fallback_dtype(c), _fallback_dtype(a), _fallback_dtype(b), beta=beta, alpha=alpha), a)


def baddbmm(c, a, b, beta=1, alpha=1):
    return _back(torch.baddbmm(_fallback_dtype(c), _fallback_dtype(a), _fallback_dtype(b), beta=beta, alpha=alpha), a)


def linear(x, w, bias=None):
    """custom_fallback_dipu_linear, CustomFallbackFunctions.hpp:417-451."""
    b = None if bias is None else _fallback_dtype(bias)
    return _back(F.linear(_fallback_dtype(x), _fallback_dtype(w), b), x)


def index_put_(x, indices, values, accumulate=False):
    """custom_fallback_dipu__index_put_impl_, CustomFallbackFunctions.hpp:78-91."""
    return x.index_put_(tuple(indices), values, accumulate=accumulate)


# ---- selection / mask / gather helpers: the generic boxed CPU fallback, i.e. stock ATen ----
# (dipu/torch_dipu/csrc_dipu/aten/RegisterDIPU.cpp:131-158). Known answers the reference's
# tests hold: dipu/tests/python/unittests/test_gather.py:10-16, test_arange.py:8-24,
# test_tri.py:9-20, test_where.py:11-31, test_masked_fill.py:8-76, test_ge.py:14-24.
def where(cond, a, b):
    return torch.where(cond, a, b)


def masked_fill(x, mask, value):
    return torch.masked_fill(x, mask, value)


def tril(x, diagonal=0):
    return torch.tril(x, diagonal)


def triu(x, diagonal=0):
    return torch.triu(x, diagonal)


def arange(start, end, step, dtype=None):
    return torch.arange(start, end, step, dtype=dtype)


def index_select(x, dim, index):
    return torch.index_select(x, dim, index.long())


def gather(x, dim, index):
    return torch.gather(x, dim, index.long())


def compare(name, a, b):
    return getattr(torch, name)(a, b)


# ---- fused ops restated from the reference's PyTorch definitions -----------
def rms_norm(x, weight, eps):
    """lightllm_rms_norm_impl, ext_ops.py:47-49 (arithmetic in x's own dtype)."""
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def rms_norm_fp32(x, weight, eps):
    """RMSNorm.forward, model.py:34-39: normalise in fp32, cast back, then scale."""
    xf = x.float()
    normed = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).type_as(x)
    return normed * weight


def rotary_emb(x, cos, sin):
    """lightllm_rotary_emb_impl, ext_ops.py:24-33: x [seq, heads, d], cos/sin [seq, d/2], half-split pairs."""
    seq_len, h, dim = x.shape
    cos = cos.view((seq_len, 1, dim // 2))
    sin = sin.view((seq_len, 1, dim // 2))
    x0 = x[:, :, 0: dim // 2]
    x1 = x[:, :, dim // 2: dim]
    o0 = x0 * cos - x1 * sin
    o1 = x0 * sin + x1 * cos
    return torch.cat((o0, o1), dim=-1)


def precompute_freqs(dim, end, theta=10000.0):
    """precompute_freqs_cis, model.py:42-47, returned as (cos, sin) of shape [end, dim/2]."""
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2)[: (dim // 2)].float() / dim))
    t = torch.arange(end)
    freqs = torch.outer(t, freqs).float()
    return torch.cos(freqs), torch.sin(freqs)


def rotary_emb_interleaved(x, cos, sin):
    """apply_rotary_emb, model.py:58-69: adjacent pairs as complex numbers times cos + i sin.
    x [..., seq, heads, d]; cos/sin [seq, d/2]."""
    xc = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
    f = torch.polar(torch.ones_like(cos.float()), torch.atan2(sin.float(), cos.float()))
    shape = [1] * xc.dim()
    shape[-3] = xc.shape[-3]
    shape[-1] = xc.shape[-1]
    out = torch.view_as_real(xc * f.view(*shape)).flatten(-2)
    return out.type_as(x)


def dest_index_copy_kv(pool, k, dest_loc):
    """out[dest_loc[i]] = k[i]: index_put on the leading dim (diopi_functions.yaml:2370-2382 semantics;
    contiguous-range form ext_ops.py:146-149)."""
    pool[dest_loc.long()] = k
    return pool


def context_attention(q, k, v, b_start_loc, b_seq_len):
    """lightllm_prompt_attention_inference_impl, ext_ops.py:62-87, applied per packed sequence.
    q [tokens, heads, d]; k, v [tokens, kv_heads, d]; fp32 scores, additive -999999999999 mask."""
    out = torch.empty_like(q)
    heads, d = q.shape[1], q.shape[2]
    kv_heads = k.shape[1]
    for s, n in zip(b_start_loc.tolist(), b_seq_len.tolist()):
        if n == 0:
            continue
        xq = q[s:s + n].view(1, n, heads, d)
        xk = k[s:s + n].view(1, n, kv_heads, d)
        xv = v[s:s + n].view(1, n, kv_heads, d)
        if kv_heads != heads:
            rep = heads // kv_heads
            xk = xk.repeat_interleave(rep, dim=2)
            xv = xv.repeat_interleave(rep, dim=2)
        mask = torch.tril(torch.ones(n, n), diagonal=0).unsqueeze(0).unsqueeze(0)
        mask = mask.masked_fill(mask == 0., -999999999999.0)
        mask = mask.masked_fill(mask == 1., 0.0)
        xq = xq.transpose(1, 2).float()
        keys = xk.transpose(1, 2).float()
        values = xv.transpose(1, 2).float()
        scores = torch.matmul(xq, keys.transpose(2, 3)) / math.sqrt(d)
        scores = F.softmax(scores + mask.float(), dim=-1).type_as(xq)
        o = torch.matmul(scores, values).transpose(1, 2).contiguous().reshape(-1, heads, d)
        out[s:s + n] = o.to(q.dtype)
    return out


def token_attention(q, k_pool, v_pool, b_loc, b_seq_len, max_input_len):
    """lightllm_flash_attention_inference_impl, ext_ops.py:100-133, with each sequence's cached
    tokens gathered from the pool through its right-aligned slot table row."""
    batch, heads, d = q.shape
    kv_heads = k_pool.shape[1]
    res = []
    for i in range(batch):
        n = int(b_seq_len[i])
        slots = b_loc[i, max_input_len - n:max_input_len].long()
        k = k_pool[slots].float()
        v = v_pool[slots].float()
        if kv_heads != heads:
            k = k.repeat_interleave(heads // kv_heads, dim=1)
            v = v.repeat_interleave(heads // kv_heads, dim=1)
        xq = q[i].float().view(heads, 1, d)
        xk = k.transpose(0, 1).transpose(1, 2)          # heads, d, n
        out = torch.bmm(xq, xk) / math.sqrt(d)          # heads, 1, n
        out = out.softmax(-1)
        xv = v.transpose(0, 1)                           # heads, n, d
        res.append(torch.bmm(out, xv).view(1, heads, d))
    return torch.cat(res).to(q.dtype)


def token_logits(q, k_pool, b_loc, b_start_loc, b_seq_len, max_input_len, total):
    """The q.K^T/sqrt(d) half of ext_ops.py:116-118 laid out [heads, total_tokens]."""
    batch, heads, d = q.shape
    kv_heads = k_pool.shape[1]
    att = torch.zeros(heads, total, dtype=torch.float32)
    for i in range(batch):
        n = int(b_seq_len[i])
        s = int(b_start_loc[i])
        slots = b_loc[i, max_input_len - n:max_input_len].long()
        k = k_pool[slots].float()
        if kv_heads != heads:
            k = k.repeat_interleave(heads // kv_heads, dim=1)
        att[:, s:s + n] = torch.einsum("hd,nhd->hn", q[i].float(), k) / math.sqrt(d)
    return att


def weight_only_int8_linear(x, w_int8, scale, bias=None):
    """out = x . (W_int8 * scale[:, None])^T computed in fp32 (the dequantised fp32 matmul)."""
    wf = w_int8.float() * scale.float()[:, None]
    out = x.float() @ wf.t()
    if bias is not None:
        out = out + bias.float()
    return out


# ---- the tiny LLaMA-style decoder block (fp32 parity workload) -------------
def decoder_block(x, p, heads, eps, theta=10000.0):
    """RMSNorm -> QKV linear -> rotary -> causal attention -> out linear -> residual ->
    RMSNorm -> SiLU-gated FFN -> residual; x [batch, seq, hidden]. Returns every intermediate.
    Structure of dicp/test/model/llama/model.py:108-200 with the half-split rotary of ext_ops.py."""
    b, s, hidden = x.shape
    d = hidden // heads
    inter = {}
    h1 = rms_norm(x, p["norm1"], eps)
    inter["norm1"] = h1
    qkv = linear(h1, p["wqkv"])
    inter["qkv"] = qkv
    q, k, v = qkv.split(hidden, dim=-1)
    cos, sin = precompute_freqs(d, s, theta)
    cos, sin = cos.to(x.dtype), sin.to(x.dtype)
    q = torch.stack([rotary_emb(q[i].reshape(s, heads, d), cos, sin) for i in range(b)])
    k = torch.stack([rotary_emb(k[i].reshape(s, heads, d), cos, sin) for i in range(b)])
    inter["q_rot"], inter["k_rot"] = q, k
    starts = torch.arange(b) * s
    lens = torch.full((b,), s)
    attn = context_attention(q.reshape(b * s, heads, d), k.reshape(b * s, heads, d),
                             v.reshape(b * s, heads, d), starts, lens)
    inter["attn"] = attn
    o = linear(attn.reshape(b, s, hidden), p["wo"])
    inter["o"] = o
    x1 = add(x, o)
    inter["res1"] = x1
    h2 = rms_norm(x1, p["norm2"], eps)
    inter["norm2"] = h2
    gate = linear(h2, p["wgate"])
    up = linear(h2, p["wup"])
    act = mul(silu(gate), up)
    inter["act"] = act
    down = linear(act, p["wdown"])
    inter["down"] = down
    out = add(x1, down)
    inter["out"] = out
    return out, inter
