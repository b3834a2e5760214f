"""Seeded sweeps over random valid shapes of the launchers around the three operators: sizes that are not
multiples of the kernels' tiles, one-element batches, padding, ragged lengths. Every case is checked against
the oracle to the operator's own bar (stated in the operator's test file)."""
import pytest
import torch

from oracle import gdn, mla, moe

pytestmark = pytest.mark.gpu


def _pick(rng, xs):
    return xs[int(torch.randint(len(xs), (1,), generator=rng))]


@pytest.mark.parametrize('seed', range(8))
def test_sparse_mla_and_selection(capi, dev, seed):
    rng = torch.Generator().manual_seed(5000 + seed)
    B, H = _pick(rng, [1, 2, 3, 5]), _pick(rng, [32, 64, 128, 256])
    page = _pick(rng, [16, 64])
    N = page * _pick(rng, [3, 9, 40])
    k = _pick(rng, [1, 31, 32, 33, 100, 257, 700])
    q, kv, _ = mla.mla_make_inputs(B, H, N, 1, generator=rng)
    scores = torch.randn(B, N, generator=rng)
    lengths = torch.randint(0, N + 1, (B,), generator=rng).int()
    lengths[0] = N
    idx = torch.empty(B, k, dtype=torch.int32, device=dev)
    capi.topk_select_launch(idx, scores.to(dev), lengths.to(dev))
    torch.cuda.synchronize()
    want_idx = mla.topk_select(scores, k, lengths)
    assert torch.equal(idx.cpu(), want_idx)
    pool, table = mla.mla_scatter_into_pool(kv, page, generator=rng)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, k), dtype=torch.uint8, device=dev)
    out = torch.full((B, H, 512), float('nan'), device=dev)
    out_p = torch.full((B, H, 512), float('nan'), device=dev)
    capi.sparse_mla_decode_launch(out, q.to(dev), kv.to(dev), idx, ws)
    capi.sparse_mla_decode_paged_launch(out_p, q.to(dev), pool.to(dev), table.to(dev), idx, ws.clone())
    torch.cuda.synchronize()
    ref = mla.sparse_mla_decode(q, kv, want_idx, out_dtype=torch.float32)
    live = (want_idx >= 0).any(dim=1)                # a request without any valid row has no defined output
    assert torch.isfinite(out[live.to(dev)]).all()
    if live.any():
        assert mla.rel_rms_error(out.cpu()[live], ref[live]) <= 2e-2
    assert torch.equal(out_p[live.to(dev)], out[live.to(dev)])


@pytest.mark.parametrize('seed', range(6))
def test_gdn_layer_chain(capi, dev, seed):
    rng = torch.Generator().manual_seed(6000 + seed)
    B = _pick(rng, [1, 2, 7, 33])
    Hqk = _pick(rng, [1, 2, 4])
    Hv = Hqk * _pick(rng, [1, 2, 4])
    dt = _pick(rng, [torch.float32, torch.bfloat16])
    L, K = _pick(rng, [(4, 4), (3, 4), (2, 3), (1, 2)])
    d = 128
    x, cstate, weight, bias = gdn.conv_make_inputs(B, Hqk * d, Hv * d, L, K, dt, generator=rng)
    _, _, _, a, b, a_log, dt_bias, state = gdn.gdn_make_raw_inputs(B, Hv, Hqk, qkv_dtype=dt, generator=rng)
    z = torch.randn(B, Hv, d, generator=rng).to(dt)
    norm_w = (1 + 0.1 * torch.randn(d, generator=rng)).to(dt)
    want_c = cstate.clone()
    mixed = gdn.causal_conv1d_update(x, want_c, weight, bias)
    q = torch.empty(B, Hqk * d, dtype=dt, device=dev)
    k = torch.empty_like(q)
    v = torch.empty(B, Hv * d, dtype=dt, device=dev)
    cs = cstate.to(dev)
    capi.causal_conv1d_update_launch(q, k, v, cs, x.to(dev), weight.to(dev), bias.to(dev))
    s = state.to(dev)
    out = torch.empty(B, Hv, d, dtype=dt, device=dev)
    capi.gdn_decode_fused_norm_launch(out, s, q.view(B, Hqk, d), k.view(B, Hqk, d), v.view(B, Hv, d), a.to(dev),
                                      b.to(dev), a_log.to(dev), dt_bias.to(dev), z.to(dev), norm_w.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(cs.cpu(), want_c)
    got_mixed = torch.cat([q, k, v], dim=1).cpu()
    assert ((got_mixed.float() - mixed.float()).abs() <= mixed.float().abs() * 2.0 ** -7 + 1e-6).all()
    want, want_s = gdn.gdn_decode_fused_norm_step(q.view(B, Hqk, d).cpu(), k.view(B, Hqk, d).cpu(),
                                                  v.view(B, Hv, d).cpu(), a, b, a_log, dt_bias, state.clone(), z, norm_w)
    assert gdn.gdn_close(s.cpu(), want_s)
    tol = 1e-3 if dt == torch.float32 else 2.0 ** -7
    assert ((out.cpu().float() - want.float()).abs() <= tol * want.float().abs() + 1e-3 * want.float().abs().max()).all()


@pytest.mark.parametrize('seed', range(6))
def test_router_chain(capi, dev, seed):
    rng = torch.Generator().manual_seed(7000 + seed)
    T = _pick(rng, [1, 5, 64, 65, 333])
    H = 64 * _pick(rng, [1, 3, 8, 33])
    G = _pick(rng, [1, 2, 4, 8])
    E = G * _pick(rng, [4, 8, 16, 32])
    kg = int(torch.randint(1, G + 1, (1,), generator=rng))
    k = min(int(torch.randint(1, 9, (1,), generator=rng)), kg * (E // G))
    x = torch.randn(T, H, generator=rng).bfloat16()
    w = torch.randn(E, H, generator=rng) * H ** -0.5
    bias = 0.1 * torch.randn(E, generator=rng)
    logits = torch.empty(T, E, device=dev)
    nbytes = capi.moe_router_logits_workspace_bytes(T, H, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev) if nbytes else None
    capi.moe_router_logits_launch(logits, x.to(dev), w.to(dev), ws)
    ids = torch.empty(T, k, dtype=torch.int32, device=dev)
    wts = torch.empty(T, k, device=dev)
    capi.moe_route_grouped_launch(ids, wts, logits, bias.to(dev), G, kg, True, 1.5)
    torch.cuda.synchronize()
    want = x.double() @ w.double().T
    assert ((logits.cpu().double() - want).abs() <= H * 2.0 ** -24 * (x.double().abs() @ w.double().abs().T) + 1e-12).all()
    # the routing is checked on the kernel's own logits, where it is exact
    want_ids, want_w, _ = moe.route_grouped(logits.cpu(), bias, k, G, kg, True, 1.5)
    same = (ids.cpu() == want_ids).all(dim=1)
    assert (~same).sum().item() <= max(1, T // 500)
    torch.testing.assert_close(wts.cpu()[same], want_w[same], rtol=1e-5, atol=1e-9)


@pytest.mark.parametrize('seed', range(8))
def test_moe_layer(capi, dev, seed):
    """The whole layer on a random valid shape, stage by stage and end to end (test_moe_gpu.check_layer states the
    bars): the streaming GEMMs, and the tiled ones (config bit 16) both with gate/up on the bf16 matrix core and as
    the layer runs them by default, e4m3 matrix core with the large codes repaired."""
    from test_moe_gpu import check_layer
    rng = torch.Generator().manual_seed(9000 + seed)
    T = _pick(rng, [1, 7, 33, 129, 300, 517])
    form = seed % 3
    H = 128 * _pick(rng, [1, 2, 3, 6]) if form == 0 else 256 * _pick(rng, [1, 2, 3])   # (the tiled GEMMs: multiples of 256)
    inter = 128 * _pick(rng, [1, 2, 4])
    E = _pick(rng, [2, 3, 5, 8])
    k = int(torch.randint(1, min(E, 4) + 1, (1,), generator=rng))
    biased = [0] if seed % 2 else None
    if form == 0:
        check_layer(capi, dev, T, H, inter, E, k, 9100 + seed, config=1, biased=biased)
    elif form == 1:
        check_layer(capi, dev, T, H, inter, E, k, 9100 + seed, config=16, biased=biased, requant='exact')
    else:
        check_layer(capi, dev, T, H, inter, E, k, 9100 + seed, config=16, biased=biased, requant='repaired')
