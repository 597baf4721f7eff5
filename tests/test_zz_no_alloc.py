"""The decode attention entry point that allocates nothing, through the C ABI, against the entry point that takes its
partial results from the context's workspace: same kernels, so the outputs are bit-identical."""
import pytest
import torch

from oracle import cpu_fallback as oracle
from tests.parity import assert_exact, assert_half

pytestmark = pytest.mark.gpu


def _case(pkg, dev, seed, batch, heads, max_len):
    w = pkg.workloads.paged_decode(seed=seed, batch=batch, heads=heads, head_dim=128, min_len=1, max_len=max_len, pool_slots=16384)
    d = {k: (v.to(dev) if hasattr(v, "to") else v) for k, v in w.items()}
    return w, d


def test_no_alloc_decode_attention_matches_the_allocating_entry_point(ops, dev, pkg):
    # two calls in a row share the device array; the second is smaller (fewer sequences, fewer splits) and must not
    # see anything the first left behind
    for seed, batch, heads, max_len in [(11, 9, 8, 5000), (12, 3, 4, 1200)]:
        w, d = _case(pkg, dev, seed, batch, heads, max_len)
        args = (d["q"], d["k_pool"], d["v_pool"], d["b_loc"], d["b_start_loc"], d["b_seq_len"], w["max_input_len"])
        want = ops.token_decode_attention(*args)
        got = torch.full_like(want, float("nan"))
        ops.token_decode_attention(*args, out=got, no_alloc=True)
        assert_exact(got, want.cpu())
        ref = oracle.token_attention(w["q"].float(), w["k_pool"].float(), w["v_pool"].float(), w["b_loc"], w["b_seq_len"], w["max_input_len"])
        assert_half(got, ref)
    # a single split uses no partial results at all
    w, d = _case(pkg, dev, 13, 5, 4, 300)
    args = (d["q"], d["k_pool"], d["v_pool"], d["b_loc"], d["b_start_loc"], d["b_seq_len"], w["max_input_len"])
    got = torch.empty_like(d["q"])
    ops.token_decode_attention(*args, out=got, no_alloc=True)
    assert_exact(got, ops.token_decode_attention(*args).cpu())


def test_no_alloc_decode_attention_requests_no_workspace_and_rejects_oversize(ops, dev, pkg):
    rt = pkg.runtime
    w, d = _case(pkg, dev, 14, 6, 8, 3000)
    args = (d["q"], d["k_pool"], d["v_pool"], d["b_loc"], d["b_start_loc"], d["b_seq_len"], w["max_input_len"])
    out = torch.empty_like(d["q"])
    ops.token_decode_attention(*args, out=out, no_alloc=True)       # first call on the device: address lookup
    torch.cuda.synchronize()
    before = rt.cachingStats()
    ops.token_decode_attention(*args, out=out, no_alloc=True)
    torch.cuda.synchronize()
    assert rt.cachingStats() == before                              # not one request reached the allocator
    scope = ops.WorkspaceScope()                                    # keeps what its ops request until close()
    with scope:
        ops.token_decode_attention(*args, out=out, no_alloc=True)
        assert rt.cachingStats()["allocations"] == before["allocations"]
        ops.token_decode_attention(*args)
        assert rt.cachingStats()["allocations"] == before["allocations"] + 1   # the allocating entry point's workspace
    torch.cuda.synchronize()
    scope.close()
    # 64 sequences x 32 heads x 64 splits x 130 floats = 68 MB of partial results: beyond the 32 MiB the library holds
    big_loc = torch.zeros(64, 40000, dtype=torch.int32, device=dev)
    q = torch.zeros(64, 32, 128, dtype=torch.bfloat16, device=dev)
    pool = torch.zeros(64, 32, 128, dtype=torch.bfloat16, device=dev)
    lens = torch.full((64,), 40000, dtype=torch.int32, device=dev)
    with pytest.raises(pkg.diopi.DiopiError, match="allocates nothing"):
        ops.token_decode_attention(q, pool, pool, big_loc, lens, lens, 40000, out=torch.empty_like(q), no_alloc=True)
    # the allocating entry point takes the same call
    ops.token_decode_attention(q, pool, pool, big_loc, lens, lens, 40000)
    torch.cuda.synchronize()
