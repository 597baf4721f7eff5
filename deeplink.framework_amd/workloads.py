"""Seeded synthetic inputs for the measured configurations (all generated on the CPU with a
torch.Generator so the device path and the CPU oracle see identical values).

  tiny_block      batch 2, seq 128, hidden 512, 8 heads x 64, FFN 1376, fp32
  memory_bound    bf16 [8192, 4096] pairs, RMSNorm weight, rotary [8192, 32, 128] + tables
  paged_decode    batch 64, 32 heads x 128, lens U[512, 4096], pool of 262144 slots
  llama7b_layer   batch 4, seq 2048, hidden 4096, 32 x 128, FFN 11008, bf16
  int8_linear     M in {1, 4, 16}, K 4096, N 11008, int8 weights, fp16 scales
Each generator takes scale-down arguments so parity tests can use small instances.
"""
import math

import torch


def _gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def rotary_tables(head_dim, positions, theta=10000.0, dtype=torch.float32):
    """cos/sin [positions, head_dim/2] for positions 0..positions-1."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2).float() / head_dim))
    ang = torch.outer(torch.arange(positions).float(), inv)
    return torch.cos(ang).to(dtype), torch.sin(ang).to(dtype)


def tiny_block(seed=0, batch=2, seq=128, hidden=512, heads=8, ffn=1376, dtype=torch.float32):
    g = _gen(seed)
    x = torch.randn(batch, seq, hidden, generator=g).to(dtype)
    w = lambda *s: (torch.randn(*s, generator=g) * 0.02).to(dtype)
    params = {
        "wqkv": w(3 * hidden, hidden), "wo": w(hidden, hidden), "wgate": w(ffn, hidden), "wup": w(ffn, hidden),
        "wdown": w(hidden, ffn), "norm1": torch.ones(hidden, dtype=dtype), "norm2": torch.ones(hidden, dtype=dtype),
    }
    return x, params, {"heads": heads, "eps": 1e-6, "theta": 10000.0}


def memory_bound(seed=0, rows=8192, cols=4096, heads=32, head_dim=128, dtype=torch.bfloat16):
    g = _gen(seed)
    a = torch.randn(rows, cols, generator=g).to(dtype)
    b = torch.randn(rows, cols, generator=g).to(dtype)
    w = (1.0 + 0.1 * torch.randn(cols, generator=g)).to(dtype)
    xr = torch.randn(rows, heads, head_dim, generator=g).to(dtype)
    cos, sin = rotary_tables(head_dim, rows, dtype=dtype)
    return {"a": a, "b": b, "rms_weight": w, "eps": 1e-5, "rot_x": xr, "cos": cos, "sin": sin}


def paged_decode(seed=0, batch=64, heads=32, head_dim=128, min_len=512, max_len=4096, pool_slots=262144,
                 dtype=torch.bfloat16, index_dtype=torch.int32, fill_pool=True):
    """Sequence b owns perm[off_b : off_b + len_b (+1 for the new token)]. Returns the pool with the
    owned slots filled N(0,1), the new token's k/v, its destination slots, and the slot table
    (right-aligned, width = max over (len_b + 1)) describing each sequence AFTER the new token."""
    g = _gen(seed)
    lens = torch.randint(min_len, max_len + 1, (batch,), generator=g)
    perm = torch.randperm(pool_slots, generator=g)
    total = int(lens.sum()) + batch
    assert total <= pool_slots, "pool too small for the requested sequences"
    new_lens = lens + 1
    width = int(new_lens.max())
    b_loc = torch.zeros(batch, width, dtype=index_dtype)
    dest = torch.empty(batch, dtype=index_dtype)
    owned = []
    off = 0
    for b in range(batch):
        n = int(new_lens[b])
        slots = perm[off:off + n]
        off += n
        b_loc[b, width - n:] = slots.to(index_dtype)
        dest[b] = slots[-1]
        owned.append(slots[:-1])
    k_pool = torch.zeros(pool_slots, heads, head_dim, dtype=dtype)
    v_pool = torch.zeros(pool_slots, heads, head_dim, dtype=dtype)
    if fill_pool:
        idx = torch.cat(owned)
        k_pool[idx] = torch.randn(idx.numel(), heads, head_dim, generator=g).to(dtype)
        v_pool[idx] = torch.randn(idx.numel(), heads, head_dim, generator=g).to(dtype)
    q = torch.randn(batch, heads, head_dim, generator=g).to(dtype)
    k_new = torch.randn(batch, heads, head_dim, generator=g).to(dtype)
    v_new = torch.randn(batch, heads, head_dim, generator=g).to(dtype)
    b_start = torch.zeros(batch, dtype=index_dtype)
    b_start[1:] = torch.cumsum(new_lens, 0)[:-1].to(index_dtype)
    return {"q": q, "k_pool": k_pool, "v_pool": v_pool, "k_new": k_new, "v_new": v_new, "dest_loc": dest,
            "b_loc": b_loc, "b_start_loc": b_start, "b_seq_len": new_lens.to(index_dtype), "max_input_len": width,
            "total_tokens": total}


def llama7b_layer(seed=0, batch=4, seq=2048, hidden=4096, heads=32, ffn=11008, dtype=torch.bfloat16):
    g = _gen(seed)
    x = torch.randn(batch, seq, hidden, generator=g).to(dtype)
    w = lambda *s: (torch.randn(*s, generator=g) * 0.02).to(dtype)
    params = {
        "wqkv": w(3 * hidden, hidden), "wo": w(hidden, hidden), "wgate": w(ffn, hidden), "wup": w(ffn, hidden),
        "wdown": w(hidden, ffn), "norm1": torch.ones(hidden, dtype=dtype), "norm2": torch.ones(hidden, dtype=dtype),
    }
    return x, params, {"heads": heads, "eps": 1e-5, "theta": 10000.0}


def int8_linear(seed=0, m=1, k=4096, n=11008, dtype=torch.bfloat16):
    g = _gen(seed)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    scale = (0.001 + 0.019 * torch.rand(n, generator=g)).to(torch.float16)
    return {"x": x, "w": w, "scale": scale}
