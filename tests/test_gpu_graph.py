"""The op library under HIP graph capture: a decode step of a decoder layer (every launch-bound op of the path, the
workspace users included) is recorded once and replayed; each replay must equal the eager result bit for bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def make_step(ops, pkg, dev):
    torch.manual_seed(11)
    batch, heads, d, hidden, ffn = 16, 8, 128, 1024, 2816
    w = pkg.workloads.paged_decode(seed=5, batch=batch, heads=heads, head_dim=d, min_len=64, max_len=1500, pool_slots=16384)
    t = {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in w.items()}
    bf = torch.bfloat16
    rnd = lambda *shape, scale=1.0: (torch.randn(*shape) * scale).to(bf).to(dev)
    p = {"x": rnd(batch, hidden), "n1": rnd(hidden) * 0.1 + 1, "n2": rnd(hidden) * 0.1 + 1,
         "wqkv": rnd(3 * hidden, hidden, scale=0.03), "wo": rnd(hidden, hidden, scale=0.03),
         "wgu": ops.interleave_gate_up(rnd(ffn, hidden, scale=0.03), rnd(ffn, hidden, scale=0.03)),
         "wdown": rnd(hidden, ffn, scale=0.03),
         "a": rnd(300, 512), "b": rnd(512, 640).t().contiguous().t()}       # a mid-size product: split-K partials
    cos, sin = pkg.workloads.rotary_tables(d, int(w["b_seq_len"].max()), dtype=torch.float32)
    at = (w["b_seq_len"] - 1).long()                                         # each sequence's new token position
    p["cos"], p["sin"] = cos[at].to(bf).to(dev), sin[at].to(bf).to(dev)
    o = {"h": torch.empty(batch, hidden, dtype=bf, device=dev), "qkv": torch.empty(batch, 3 * hidden, dtype=bf, device=dev),
         "q": torch.empty(batch, heads, d, dtype=bf, device=dev), "k": torch.empty(batch, heads, d, dtype=bf, device=dev),
         "v": torch.empty(batch, heads, d, dtype=bf, device=dev), "att": torch.empty(batch, heads, d, dtype=bf, device=dev),
         "o": torch.empty(batch, hidden, dtype=bf, device=dev), "x1": torch.empty(batch, hidden, dtype=bf, device=dev),
         "h2": torch.empty(batch, hidden, dtype=bf, device=dev), "act": torch.empty(batch, ffn, dtype=bf, device=dev),
         "down": torch.empty(batch, hidden, dtype=bf, device=dev), "y": torch.empty(batch, hidden, dtype=bf, device=dev),
         "ab": torch.empty(300, 640, dtype=bf, device=dev), "sm": torch.empty(640, 300, dtype=bf, device=dev)}

    def step():
        ops.rms_norm(p["x"], p["n1"], 1e-5, out=o["h"])
        ops.linear(o["h"], p["wqkv"], out=o["qkv"])
        qv, kv, vv = (o["qkv"][:, i * hidden:(i + 1) * hidden].reshape(batch, heads, d) for i in range(3))
        ops.rotary_emb(qv, p["cos"], p["sin"], out=o["q"])
        ops.rotary_emb(kv, p["cos"], p["sin"], out=o["k"])
        ops.copy_(o["v"], vv)
        ops.dest_index_copy_kv(o["k"], t["dest_loc"], t["k_pool"])
        ops.dest_index_copy_kv(o["v"], t["dest_loc"], t["v_pool"])
        ops.token_decode_attention(o["q"], t["k_pool"], t["v_pool"], t["b_loc"], t["b_start_loc"], t["b_seq_len"],
                                   t["max_input_len"], out=o["att"])
        ops.linear(o["att"].reshape(batch, hidden), p["wo"], out=o["o"])
        ops.add(p["x"], o["o"], out=o["x1"])
        ops.rms_norm(o["x1"], p["n2"], 1e-5, out=o["h2"])
        ops.linear_silu_mul(o["h2"], p["wgu"], out=o["act"])
        ops.linear(o["act"], p["wdown"], out=o["down"])
        ops.add(o["x1"], o["down"], out=o["y"])
        ops.mm(p["a"], p["b"], out=o["ab"])                                  # transposed operand + split-K workspace
        ops.softmax(o["ab"].t(), 1, out=o["sm"])                             # dense copy of a strided input

    return p, o, step


def test_decode_step_replays_from_a_hip_graph(ops, dev, pkg):
    p, o, step = make_step(ops, pkg, dev)
    inputs = [(torch.randn(p["x"].shape) * s).to(torch.bfloat16).to(dev) for s in (1.0, 0.5, 2.0, 1.5)]
    want = []
    for x in inputs:                                                         # eager results, one per input
        p["x"].copy_(x)
        step()
        torch.cuda.synchronize()
        want.append({k: v.clone() for k, v in o.items()})
    assert not torch.equal(want[0]["y"], want[1]["y"])

    side = torch.cuda.Stream()                                               # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        # recording may not allocate device memory: passes that hold all their workspace, as the recording will,
        # until one is served from the capture stream's cache alone (the next pass then repeats its choices)
        for _ in range(6):
            before = pkg.runtime.cachingStats()["num_device_malloc"]
            warm = ops.WorkspaceScope()
            with warm:
                step()
            side.synchronize()
            warm.close()
            if pkg.runtime.cachingStats()["num_device_malloc"] == before:
                break
        else:
            pytest.fail("the workspace cache did not reach a steady state")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        scope = ops.WorkspaceScope()
        with scope:
            step()
    assert scope.ctx.workspace()[0] >= 3                                     # the workspace users are in the graph
    torch.cuda.synchronize()
    for v in o.values():
        v.zero_()
    scratch = torch.randn(64, 48, device=dev).t()
    for round_ in range(2):
        for x, ref in zip(inputs, want):
            p["x"].copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            for name, r in ref.items():
                assert torch.equal(o[name], r), f"replay differs from eager in {name} (pass {round_})"
            # eager work of the same library between replays, with a workspace of its own, and a sync
            assert torch.allclose(ops.softmax(scratch, 1).cpu(), torch.softmax(scratch.cpu(), 1), atol=1e-6)
            torch.cuda.synchronize()
    del graph
    scope.close()


def test_workspace_request_during_capture_is_served_from_the_cache_or_refused(ops, dev, pkg):
    """While a stream is being captured a workspace request may not reach hipMalloc: a block cached for that stream is
    handed out, anything else is an error that says what to do, raised before any HIP call is made."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    x = torch.randn(333, 777, device=dev).t()                                # strided input: softmax copies it densely
    out = torch.empty(777, 333, device=dev)
    big = torch.randn(2222, 3333, device=dev).t()                            # a size nothing has cached
    big_out = torch.empty(3333, 2222, device=dev)
    with torch.cuda.stream(side):
        warm = ops.WorkspaceScope()
        with warm:
            ops.softmax(x, 1, out=out)
        side.synchronize()
        warm.close()                                                         # the block is now cached for `side`
    mallocs = pkg.runtime.cachingStats()["num_device_malloc"]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        scope = ops.WorkspaceScope()
        with scope:
            ops.softmax(x, 1, out=out)                                       # served from the cache
            with pytest.raises(pkg.diopi.DiopiError, match="captured into a graph"):
                ops.softmax(big, 1, out=big_out)
    assert pkg.runtime.cachingStats()["num_device_malloc"] == mallocs
    out.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.allclose(out.cpu(), torch.softmax(x.cpu(), 1), atol=1e-6)
    del graph
    scope.close()
