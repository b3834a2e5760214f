"""One decode step of each operator captured in a HIP graph and replayed.

The launchers take a stream, allocate nothing and record no memset, so a step can be captured by a
caller (a serving loop that replays a decode graph). Every replay is checked against the eager result,
with eager work and synchronisations between the replays."""
import pytest
import torch

from oracle import gdn, mla, moe

pytestmark = pytest.mark.gpu


def capture(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()                                   # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        fn()
    return graph


def eager_noise(dev):
    # unrelated eager work between replays
    a = torch.randn(512, 512, device=dev)
    (a @ a).sum().item()


def test_gdn_decode_steps_in_a_graph(capi, dev):
    gen = torch.Generator().manual_seed(5)
    ins = gdn.gdn_make_inputs(4, 8, 4, qkv_dtype=torch.bfloat16, generator=gen)
    q, k, v, g, beta, state0 = (t.to(dev) for t in ins)
    state = state0.clone()
    o = torch.empty(4, 8, 128, device=dev)
    graph = capture(lambda: capi.gdn_decode_launch(o, state, q, k, v, g, beta))
    state.copy_(state0)                         # capture and warm-up advanced the state
    ref_state = state0.clone()
    ref_o = torch.empty_like(o)
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        capi.gdn_decode_launch(ref_o, ref_state, q, k, v, g, beta)   # eager, same step
        torch.cuda.synchronize()
        assert torch.equal(o, ref_o) and torch.equal(state, ref_state)
        eager_noise(dev)
    want_o, want_s = gdn.gdn_decode_step(*ins[:5], ins[5].clone())
    for _ in range(2):
        want_o, want_s = gdn.gdn_decode_step(*ins[:5], want_s)
    assert gdn.gdn_close(o.cpu(), want_o) and gdn.gdn_close(state.cpu(), want_s)


def test_sparse_mla_decode_in_a_graph(capi, dev):
    gen = torch.Generator().manual_seed(6)
    q, kv, idx = (t.to(dev) for t in mla.mla_make_inputs(2, 128, 600, 160, generator=gen))
    ws = torch.empty(capi.sparse_mla_workspace_bytes(2, 128, 160), dtype=torch.uint8, device=dev)
    out = torch.empty(2, 128, 512, device=dev, dtype=torch.bfloat16)
    graph = capture(lambda: capi.sparse_mla_decode_launch(out, q, kv, idx, ws))
    eager = torch.empty_like(out)
    ws2 = torch.empty_like(ws)
    for r in range(3):
        if r:                                   # new inputs in the captured buffers
            q.copy_(torch.randn(q.shape, device=dev).bfloat16())
            idx.copy_(torch.stack([torch.randperm(600, device=dev)[:160] for _ in range(2)]).int())
        out.fill_(float('nan'))
        graph.replay()
        torch.cuda.synchronize()
        capi.sparse_mla_decode_launch(eager, q, kv, idx, ws2)
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        eager_noise(dev)
    ref = mla.sparse_mla_decode(q, kv, idx, out_dtype=torch.float32)
    assert mla.rel_rms_error(out.float(), ref) <= 2e-2 + mla.rel_rms_error(ref.bfloat16().float(), ref)


def test_moe_decode_layer_in_a_graph(capi, dev):
    T, H, I, E, k = 24, 512, 256, 16, 4
    gen = torch.Generator().manual_seed(7)
    w13_q, w13_s, w2_q, w2_s = (t.to(dev) for t in moe.moe_make_weights(E, H, I, generator=gen))
    x, logits = (t.to(dev) for t in moe.moe_make_inputs(T, H, E, generator=gen))
    ws = torch.empty(capi.moe_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=dev)
    out = torch.empty(T, H, device=dev, dtype=torch.bfloat16)
    graph = capture(lambda: capi.moe_fp8_launch(out, x, logits, w13_q, w13_s, w2_q, w2_s, ws, top_k=k))
    eager = torch.empty_like(out)
    ws2 = torch.empty_like(ws)
    for r in range(3):
        if r:
            x.copy_(torch.randn(T, H, device=dev).bfloat16())
            logits.copy_(torch.randn(T, E, device=dev))
        out.fill_(float('nan'))
        graph.replay()
        torch.cuda.synchronize()
        capi.moe_fp8_launch(eager, x, logits, w13_q, w13_s, w2_q, w2_s, ws2, top_k=k)
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        eager_noise(dev)
