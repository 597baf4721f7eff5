"""The decoder block of the parity workloads expressed through the op adapter (device path).
Mirrors oracle.cpu_fallback.decoder_block step for step so every intermediate can be compared."""
import torch


def run_decoder_block(ops, x, p, cfg, fused_ffn=False, stacked_gate_up=False, fused_rotary=False):
    heads, eps, theta = cfg["heads"], cfg["eps"], cfg["theta"]
    b, s, hidden = x.shape
    d = hidden // heads
    inter = {}
    h1 = ops.rms_norm(x, p["norm1"], eps)
    inter["norm1"] = h1
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    ang = torch.outer(torch.arange(s, dtype=torch.float32), inv)
    cos, sin = torch.cos(ang).to(x.dtype).to(x.device), torch.sin(ang).to(x.dtype).to(x.device)
    if fused_rotary:
        # q and k leave the stacked projection rotated (adjacent-pair form on weight rows permuted at load time);
        # their head dims are then a fixed permutation of the half-split results, which attention does not see
        w = torch.cat([ops.interleave_rotary_rows(p["wqkv"][:hidden], d), ops.interleave_rotary_rows(p["wqkv"][hidden:2 * hidden], d),
                       p["wqkv"][2 * hidden:]], dim=0)
        qkv = ops.linear_rotary(h1, w, cos, sin, 2 * hidden, d, interleaved=True)
        q, k, v = qkv.split(hidden, dim=-1)
        q, k = q.reshape(b, s, heads, d), k.reshape(b, s, heads, d)
        unperm = lambda t: t.reshape(b, s, heads, d // 2, 2).transpose(3, 4).reshape(b, s, heads, d)
        inter["qkv"] = torch.cat([unperm(q).reshape(b, s, hidden), unperm(k).reshape(b, s, hidden), v], dim=-1)  # rotated q, k
        inter["q_rot"], inter["k_rot"] = unperm(q), unperm(k)
    else:
        qkv = ops.linear(h1, p["wqkv"])
        inter["qkv"] = qkv
        q, k, v = qkv.split(hidden, dim=-1)  # strided views: the rotary kernel sees non-contiguous input
        q = ops.rotary_emb(q.reshape(b, s, heads, d), cos, sin)
        k = ops.rotary_emb(k.reshape(b, s, heads, d), cos, sin)
        inter["q_rot"], inter["k_rot"] = q, k
    starts = (torch.arange(b, dtype=torch.int32) * s).to(x.device)
    lens = torch.full((b,), s, dtype=torch.int32).to(x.device)
    vv = v.reshape(b * s, heads, d).contiguous()
    attn = ops.context_attention(q.reshape(b * s, heads, d), k.reshape(b * s, heads, d), vv, starts, lens, s)
    inter["attn"] = attn
    o = ops.linear(attn.reshape(b, s, hidden), p["wo"])
    inter["o"] = o
    x1 = ops.add(x, o)
    inter["res1"] = x1
    h2 = ops.rms_norm(x1, p["norm2"], eps)
    inter["norm2"] = h2
    if stacked_gate_up == "interleaved":  # both projections and the gate in one launch
        act = ops.linear_silu_mul(h2, ops.interleave_gate_up(p["wgate"], p["wup"]))
        gate = up = None
    elif stacked_gate_up:  # one projection with the two weights stacked; gate and up are its column halves (strided views)
        ffn = p["wgate"].shape[0]
        gu = ops.linear(h2, torch.cat([p["wgate"], p["wup"]], dim=0))
        gate, up = gu[..., :ffn], gu[..., ffn:]
    else:
        gate = ops.linear(h2, p["wgate"])
        up = ops.linear(h2, p["wup"])
    if gate is not None:
        act = ops.silu_mul(gate, up) if fused_ffn else ops.mul(ops.silu(gate), up)
    inter["act"] = act
    down = ops.linear(act, p["wdown"])
    inter["down"] = down
    out = ops.add(x1, down)
    inter["out"] = out
    return out, inter


def run_decomposed_decoder_block(ops, x, p, cfg):
    """The same block written the way model code without fused ext ops writes it, every step a primitive aten op
    that reaches a diopi* entry point: RMSNorm as pow / mean / add / rsqrt / mul (dicp/test/model/llama/model.py:34-39),
    rotary as arange / outer product / cos / sin / neg / cat / mul / add (half-split form of
    dicp/dicp/vendor/AscendGraph/ext_ops.py:24-33), attention as bmm / div / masked_fill / softmax / bmm with the
    causal mask built from arange and a comparison. No tensor leaves the device."""
    heads, eps, theta = cfg["heads"], cfg["eps"], cfg["theta"]
    b, s, hidden = x.shape
    d = hidden // heads
    dev = x.device

    def rms(t, w):
        var = ops.mean(ops.pow(t, 2), [-1], keepdim=True)
        return ops.mul(ops.mul(t, ops.rsqrt(ops.add(var, eps))), w)

    # rotary tables on the device: inv_freq = theta ** (-2i / d) = exp(-(ln theta) * 2i / d)
    import math
    idx = ops.arange(0, d, 2, dtype=torch.float32, device=dev)
    inv = ops.exp(ops.mul(idx, -math.log(theta) / d))
    pos = ops.arange(0, s, 1, dtype=torch.float32, device=dev)
    ang = ops.mul(pos[:, None], inv[None, :])                     # outer product by broadcasting

    def cast(t):                                                  # dtype cast through diopiCopyInp
        if t.dtype == x.dtype:
            return t
        out = torch.empty(t.shape, dtype=x.dtype, device=dev)
        ops.copy_(out, t)
        return out

    cos = cast(ops.cos(ang))[None, :, None, :]                    # [1, s, 1, d/2]
    sin = cast(ops.sin(ang))[None, :, None, :]

    def rope(t):                                                  # t [b, s, heads, d]
        t0, t1 = t[..., : d // 2], t[..., d // 2:]
        return ops.cat([ops.sub(ops.mul(t0, cos), ops.mul(t1, sin)), ops.add(ops.mul(t0, sin), ops.mul(t1, cos))], dim=-1)

    h1 = rms(x, p["norm1"])
    qkv = ops.linear(h1, p["wqkv"])
    q, k, v = (t.reshape(b, s, heads, d) for t in qkv.split(hidden, dim=-1))
    q, k = rope(q), rope(k)

    def heads_first(t):                                           # [b, s, heads, d] -> [b*heads, s, d], dense
        out = torch.empty(b, heads, s, d, dtype=t.dtype, device=dev)
        ops.copy_(out, t.permute(0, 2, 1, 3))
        return out.view(b * heads, s, d)

    qh, kh, vh = heads_first(q), heads_first(k), heads_first(v)
    kt = torch.empty(b * heads, d, s, dtype=x.dtype, device=dev)
    ops.copy_(kt, kh.transpose(1, 2))
    scores = ops.div(ops.bmm(qh, kt), math.sqrt(d))
    ids = ops.arange(0, s, 1, dtype=torch.int64, device=dev)
    future = ops.gt(ids[None, :], ids[:, None])                   # key index > query index
    probs = ops.softmax(ops.masked_fill(scores, future, float("-inf")), -1)
    ctx = ops.bmm(probs, vh).view(b, heads, s, d)
    attn = torch.empty(b, s, heads, d, dtype=x.dtype, device=dev)
    ops.copy_(attn, ctx.permute(0, 2, 1, 3))
    x1 = ops.add(x, ops.linear(attn.view(b, s, hidden), p["wo"]))
    h2 = rms(x1, p["norm2"])
    act = ops.mul(ops.silu(ops.linear(h2, p["wgate"])), ops.linear(h2, p["wup"]))
    return ops.add(x1, ops.linear(act, p["wdown"]))
