"""The decoder block of the parity workloads expressed through the op adapter (device path).
Mirrors oracle.cpu_fallback.decoder_block step for step so every intermediate can be compared."""
import torch


def run_decoder_block(ops, x, p, cfg, fused_ffn=False):
    heads, eps, theta = cfg["heads"], cfg["eps"], cfg["theta"]
    b, s, hidden = x.shape
    d = hidden // heads
    inter = {}
    h1 = ops.rms_norm(x, p["norm1"], eps)
    inter["norm1"] = h1
    qkv = ops.linear(h1, p["wqkv"])
    inter["qkv"] = qkv
    q, k, v = qkv.split(hidden, dim=-1)  # strided views: the rotary kernel sees non-contiguous input
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    ang = torch.outer(torch.arange(s, dtype=torch.float32), inv)
    cos, sin = torch.cos(ang).to(x.dtype).to(x.device), torch.sin(ang).to(x.dtype).to(x.device)
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
    gate = ops.linear(h2, p["wgate"])
    up = ops.linear(h2, p["wup"])
    act = ops.silu_mul(gate, up) if fused_ffn else ops.mul(ops.silu(gate), up)
    inter["act"] = act
    down = ops.linear(act, p["wdown"])
    inter["down"] = down
    out = ops.add(x1, down)
    inter["out"] = out
    return out, inter
