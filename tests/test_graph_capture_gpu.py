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


def test_layer_decode_chain_in_a_graph(capi, dev):
    # convolution update -> fused GDN step, both states advancing in place across replays
    gen = torch.Generator().manual_seed(8)
    B, Hv, Hqk, d = 4, 8, 4, 128
    x, cstate0, weight, bias = (t.to(dev) for t in gdn.conv_make_inputs(B, Hqk * d, Hv * d, 3, 4, torch.bfloat16,
                                                                         generator=gen))
    _, _, _, a, b, a_log, dt_bias, state0 = (t.to(dev) for t in gdn.gdn_make_raw_inputs(
        B, Hv, Hqk, qkv_dtype=torch.bfloat16, generator=gen))

    def buffers():
        return dict(q=torch.empty(B, Hqk * d, dtype=torch.bfloat16, device=dev),
                    k=torch.empty(B, Hqk * d, dtype=torch.bfloat16, device=dev),
                    v=torch.empty(B, Hv * d, dtype=torch.bfloat16, device=dev),
                    cstate=cstate0.clone(), state=state0.clone(), o=torch.empty(B, Hv, d, device=dev))

    def step(t):
        capi.causal_conv1d_update_launch(t['q'], t['k'], t['v'], t['cstate'], x, weight, bias)
        capi.gdn_decode_fused_launch(t['o'], t['state'], t['q'].view(B, Hqk, d), t['k'].view(B, Hqk, d),
                                     t['v'].view(B, Hv, d), a, b, a_log, dt_bias)

    g, e = buffers(), buffers()
    graph = capture(lambda: step(g))
    g['cstate'].copy_(cstate0)
    g['state'].copy_(state0)
    for r in range(3):
        x.copy_(torch.randn(x.shape, device=dev).bfloat16())
        graph.replay()
        torch.cuda.synchronize()
        step(e)
        torch.cuda.synchronize()
        for name in ('q', 'k', 'v', 'cstate', 'state', 'o'):
            assert torch.equal(g[name], e[name]), (r, name)
        eager_noise(dev)


def test_selection_and_paged_attention_in_a_graph(capi, dev):
    gen = torch.Generator().manual_seed(9)
    B, H, N, k, page = 2, 128, 1024, 256, 64
    q, kv, _ = mla.mla_make_inputs(B, H, N, k, generator=gen)
    pool, table = mla.mla_scatter_into_pool(kv, page, generator=gen)
    q, pool, table = q.to(dev), pool.to(dev), table.to(dev)
    scores = torch.randn(B, N, device=dev)
    lengths = torch.tensor([N, 300], dtype=torch.int32, device=dev)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, k), dtype=torch.uint8, device=dev)

    def step(idx, out, ws):
        capi.topk_select_launch(idx, scores, lengths)
        capi.sparse_mla_decode_paged_launch(out, q, pool, table, idx, ws)

    idx_g, idx_e = (torch.empty(B, k, dtype=torch.int32, device=dev) for _ in range(2))
    out_g, out_e = (torch.empty(B, H, 512, dtype=torch.bfloat16, device=dev) for _ in range(2))
    graph = capture(lambda: step(idx_g, out_g, ws))
    ws_e = torch.empty_like(ws)
    for r in range(3):
        scores.copy_(torch.randn(B, N, device=dev))
        out_g.fill_(float('nan'))
        graph.replay()
        torch.cuda.synchronize()
        step(idx_e, out_e, ws_e)
        torch.cuda.synchronize()
        assert torch.equal(idx_g, idx_e) and torch.equal(out_g, out_e)
        assert torch.equal(idx_g.cpu(), mla.topk_select(scores.cpu(), k, lengths.cpu()))
        eager_noise(dev)


def test_moe_layer_with_shared_expert_in_a_graph(capi, dev):
    T, H, I, E, k = 24, 512, 256, 16, 4
    gen = torch.Generator().manual_seed(10)
    w = [t.to(dev) for t in moe.moe_make_weights(E, H, I, gen)]
    sw = [t[0].contiguous().to(dev) for t in moe.moe_make_weights(1, H, I, gen)]
    x, logits = (t.to(dev) for t in moe.moe_make_inputs(T, H, E, gen))
    ws = torch.empty(capi.moe_shared_workspace_bytes(T, H, I, I, E, k), dtype=torch.uint8, device=dev)
    out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    graph = capture(lambda: capi.moe_fp8_shared_launch(out, x, logits, *w, *sw, ws, top_k=k))
    eager = torch.empty_like(out)
    ws2 = torch.empty_like(ws)
    for r in range(3):
        if r:
            x.copy_(torch.randn(T, H, device=dev).bfloat16())
            logits.copy_(torch.randn(T, E, device=dev))
        out.fill_(float('nan'))
        graph.replay()
        torch.cuda.synchronize()
        capi.moe_fp8_shared_launch(eager, x, logits, *w, *sw, ws2, top_k=k)
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        eager_noise(dev)


def test_fp8_indexer_chain_in_a_graph(capi, dev):
    # the new token's index key is quantised into the e4m3 key cache, then scores -> selection -> attention
    gen = torch.Generator().manual_seed(19)
    B, H, Hi, N, k = 2, 128, 64, 1024, 256
    q, kv, _ = mla.mla_make_inputs(B, H, N, k, generator=gen)
    q, kv = q.to(dev), kv.to(dev)
    keys = (torch.randn(B, N, 128, generator=gen) * 2).bfloat16().to(dev)
    codes = torch.zeros(B, N, 128, dtype=torch.uint8, device=dev)
    kscale = torch.ones(B, N, device=dev)
    capi.moe_quant_bf16_launch(codes.view(B * N, 128), kscale.view(B * N, 1), keys.view(B * N, 128))
    q_idx = torch.randn(B, Hi, 128, generator=gen).to(torch.float8_e4m3fn).view(torch.uint8).to(dev)
    w = (torch.randn(B, Hi, generator=gen) / 8).to(dev)
    lengths = torch.tensor([N, 700], dtype=torch.int32, device=dev)
    new_key = torch.empty(B, 128, dtype=torch.bfloat16, device=dev)
    new_codes = torch.empty(B, 128, dtype=torch.uint8, device=dev)
    new_scale = torch.empty(B, 1, device=dev)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, k), dtype=torch.uint8, device=dev)

    def step(scores, idx, out, ws):
        capi.moe_quant_bf16_launch(new_codes, new_scale, new_key)
        codes[:, 5].copy_(new_codes)                         # position 5 of every request takes the new key
        kscale[:, 5].copy_(new_scale[:, 0])
        capi.mla_index_scores_fp8_launch(scores, q_idx, codes, kscale, w, lengths)
        capi.topk_select_launch(idx, scores, lengths)
        capi.sparse_mla_decode_launch(out, q, kv, idx, ws)

    sc_g, sc_e = (torch.empty(B, N, device=dev) for _ in range(2))
    idx_g, idx_e = (torch.empty(B, k, dtype=torch.int32, device=dev) for _ in range(2))
    out_g, out_e = (torch.empty(B, H, 512, dtype=torch.bfloat16, device=dev) for _ in range(2))
    new_key.copy_(torch.randn(B, 128, device=dev))
    graph = capture(lambda: step(sc_g, idx_g, out_g, ws))
    ws_e = torch.empty_like(ws)
    for r in range(3):
        new_key.copy_(torch.randn(B, 128, device=dev) * (r + 1))
        out_g.fill_(float('nan'))
        graph.replay()
        torch.cuda.synchronize()
        step(sc_e, idx_e, out_e, ws_e)
        torch.cuda.synchronize()
        assert torch.equal(sc_g, sc_e) and torch.equal(idx_g, idx_e) and torch.equal(out_g, out_e)
        want = mla.index_scores_fp8(q_idx.cpu(), codes.cpu(), kscale.cpu(), w.cpu(), lengths.cpu())
        live = torch.isfinite(want)
        torch.testing.assert_close(sc_g.cpu()[live], want[live], rtol=2e-3, atol=2e-3)
        assert torch.equal(idx_g.cpu(), mla.topk_select(sc_g.cpu(), k, lengths.cpu()))
        eager_noise(dev)


def test_fp8_latent_cache_step_in_a_graph(capi, dev):
    # the new token's latent row is quantised into the e4m3 latent cache, then attended over that cache (the split
    # kernel dequantises its tiles in LDS: nothing is allocated, cleared or carried over between launches)
    gen = torch.Generator().manual_seed(23)
    B, H, N, k = 2, 128, 1024, 256
    q, kv, idx = mla.mla_make_inputs(B, H, N, k, generator=gen)
    idx[:, 0] = 9                                            # the row the step writes is always selected
    idx[1, 4] = -1
    q, kv, idx = q.to(dev), kv.to(dev), idx.to(dev)
    cache = torch.empty(B, N, capi.LATENT_ROW_BYTES, dtype=torch.uint8, device=dev)
    capi.mla_latent_quant_launch(cache, kv)
    new_row = torch.empty(B, 1, 576, dtype=torch.bfloat16, device=dev)
    new_bytes = torch.empty(B, 1, capi.LATENT_ROW_BYTES, dtype=torch.uint8, device=dev)
    ws = torch.empty(capi.sparse_mla_fp8_workspace_bytes(B, H, k), dtype=torch.uint8, device=dev)

    def step(out, ws):
        capi.mla_latent_quant_launch(new_bytes, new_row)
        cache[:, 9].copy_(new_bytes[:, 0])
        capi.sparse_mla_decode_fp8_launch(out, q, cache, idx, ws)

    out_g, out_e = (torch.empty(B, H, 512, device=dev) for _ in range(2))
    new_row.copy_(torch.randn(B, 1, 576, device=dev))
    graph = capture(lambda: step(out_g, ws))
    ws_e = torch.empty_like(ws)
    for r in range(3):
        new_row.copy_(torch.randn(B, 1, 576, device=dev) * (r + 1))
        out_g.fill_(float('nan'))
        graph.replay()
        torch.cuda.synchronize()
        step(out_e, ws_e)
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e)
        want = mla.sparse_mla_decode_fp8(q.cpu(), cache.cpu(), idx.cpu(), out_dtype=torch.float32)
        assert mla.rel_rms_error(out_g.cpu(), want) <= 2e-2
        eager_noise(dev)
