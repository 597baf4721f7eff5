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
    # 64 sequences x 32 heads x 79 splits x 130 floats = 84 MB of partial results: beyond the 32 MiB the library holds
    big_loc = torch.zeros(64, 40000, dtype=torch.int32, device=dev)
    q = torch.zeros(64, 32, 128, dtype=torch.bfloat16, device=dev)
    pool = torch.zeros(64, 32, 128, dtype=torch.bfloat16, device=dev)
    lens = torch.full((64,), 40000, dtype=torch.int32, device=dev)
    with pytest.raises(pkg.diopi.DiopiError, match="allocates nothing"):
        ops.token_decode_attention(q, pool, pool, big_loc, lens, lens, 40000, out=torch.empty_like(q), no_alloc=True)
    # the allocating entry point takes the same call
    ops.token_decode_attention(q, pool, pool, big_loc, lens, lens, 40000)
    torch.cuda.synchronize()


def test_no_alloc_decode_attention_recorded_into_a_graph_and_replayed(ops, dev, pkg):
    """What the entry point is for: after one eager call on the device (the address lookup), the call is recorded into a
    HIP graph with no workspace scope at all and replayed; every replay, with eager work and synchronizations between
    them, equals the eager result bit for bit, also after the inputs changed in place."""
    w, d = _case(pkg, dev, 15, 7, 8, 4000)
    args = (d["q"], d["k_pool"], d["v_pool"], d["b_loc"], d["b_start_loc"], d["b_seq_len"], w["max_input_len"])
    want = ops.token_decode_attention(*args)                    # eager: also warms the address lookup
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    out = torch.full_like(want, float("nan"))
    mallocs = pkg.runtime.cachingStats()["num_device_malloc"]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ops.token_decode_attention(*args, out=out, no_alloc=True)
    assert pkg.runtime.cachingStats()["num_device_malloc"] == mallocs
    for i in range(3):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert_exact(out, want)
        # eager work of the same kind between replays (it uses the same device array)
        ops.token_decode_attention(*args, out=torch.empty_like(want), no_alloc=True)
        torch.cuda.synchronize()
    d["q"].mul_(0.5)                                            # same buffers, new values
    want2 = ops.token_decode_attention(*args)
    graph.replay()
    torch.cuda.synchronize()
    assert_exact(out, want2)
    del graph
