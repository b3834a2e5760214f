"""Pins the MoE oracle: e4m3 codec, routing/sort, and the GEMM/combine arithmetic."""
import numpy as np
import pytest
import torch

from oracle import moe


def test_decode_table_matches_torch_and_closed_form():
    tab = moe.e4m3_decode_table()
    t = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(tab), np.isnan(t))
    assert np.array_equal(tab[~np.isnan(tab)], t[~np.isnan(t)])
    assert np.isnan(tab[0x7F]) and np.isnan(tab[0xFF]) and np.isnan(tab).sum() == 2
    assert tab[0x7E] == 448.0 and tab[0x38] == 1.0 and tab[0x01] == 2.0 ** -9 and tab[0x08] == 2.0 ** -6


def test_encoder_matches_torch_cast_on_values_midpoints_and_random():
    tab = moe.e4m3_decode_table()
    vals = np.sort(tab[~np.isnan(tab)])
    mids = (vals[:-1].astype(np.float64) + vals[1:]) / 2
    rng = np.random.default_rng(0)
    probe = np.concatenate([vals, mids.astype(np.float32), np.nextafter(mids.astype(np.float32), 1e9),
                            np.nextafter(mids.astype(np.float32), -1e9),
                            rng.standard_normal(200000).astype(np.float32) * 100,
                            rng.standard_normal(50000).astype(np.float32) * 0.01,
                            np.array([449, 464, 465, 480, 1e6, -1e6, 0.0, -0.0], dtype=np.float32)])
    got = moe.e4m3_encode(probe)
    want = torch.from_numpy(probe).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got, want)
    # known answers (round half to even, saturation, subnormals)
    ka = {448.0: 0x7E, 500.0: 0x7E, 17.0: 0x58, 18.0: 0x59, 1.0: 0x38, 0.25: 0x28, 2.0 ** -10: 0x00,
          3 * 2.0 ** -10: 0x02, 9.7e-4: 0x00, -1.0: 0xB8}
    for v, code in ka.items():
        assert moe.e4m3_encode(np.float32(v)) == code, v


def test_encode_decode_idempotent():
    tab = moe.e4m3_decode_table()
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    assert np.array_equal(moe.e4m3_encode(tab[codes]) & 0x7F, codes & 0x7F)


def test_group_quantisation_properties():
    gen = torch.Generator().manual_seed(1)
    v = torch.randn(6, 384, generator=gen) * 3
    v[2, 128:256] = 0                                   # an all-zero group
    q, s = moe.quantize_groups(v)
    assert q.shape == (6, 384) and s.shape == (6, 3)
    g = q.float().reshape(6, 3, 128).abs().amax(-1)
    nonzero = v.reshape(6, 3, 128).abs().amax(-1) > 0
    assert torch.all(g[nonzero] == 448.0)               # the group maximum maps to +-448
    assert torch.all(q.float()[2, 128:256] == 0) and s[2, 1] == pytest.approx(1e-12 / 448)
    back = moe.dequantize_groups(q, s)
    assert ((back - v).abs() <= v.reshape(6, 3, 128).abs().amax(-1).repeat_interleave(128, 1) / 448 * 16 + 1e-9).all()
    q2, s2 = moe.quantize_groups(back)                  # idempotent on its own output
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8))


def test_routing_against_topk_and_brute_force():
    gen = torch.Generator().manual_seed(2)
    logits = torch.randn(50, 256, generator=gen)
    ids, w = moe.route(logits)
    vals, idx = torch.topk(logits, 8, dim=-1)           # distinct floats: same order
    assert torch.equal(ids.long(), idx)
    torch.testing.assert_close(w.sum(-1), torch.ones(50))
    s = torch.sigmoid(vals)
    torch.testing.assert_close(w, s / s.sum(-1, keepdim=True))
    for t in range(5):                                  # brute force
        order = sorted(range(256), key=lambda e: (-logits[t, e].item(), e))[:8]
        assert ids[t].tolist() == order
    assert all(len(set(r)) == 8 for r in ids.tolist())


def test_routing_ties_go_to_lower_id():
    logits = torch.zeros(2, 16)
    logits[0, [3, 9, 12]] = 1.0
    logits[1, 5] = -0.0
    ids, _ = moe.route(logits, top_k=4)
    assert ids[0].tolist() == [3, 9, 12, 0] and ids[1].tolist() == [0, 1, 2, 3]


def test_sort_is_a_stable_counting_sort():
    gen = torch.Generator().manual_seed(3)
    ids, _ = moe.route(torch.randn(300, 32, generator=gen), top_k=4)
    sp, pos, off = moe.sort_pairs(ids, 32)
    flat = ids.reshape(-1)
    assert sorted(sp.tolist()) == list(range(1200))
    assert torch.equal(pos[sp.long()].long(), torch.arange(1200))
    assert off[0] == 0 and off[-1] == 1200
    assert torch.equal((off[1:] - off[:-1]).long(), torch.bincount(flat.long(), minlength=32))
    for e in range(32):
        seg = sp[off[e]:off[e + 1]]
        assert torch.all(flat[seg.long()] == e)
        assert torch.all(seg[1:] > seg[:-1])            # stable: ascending flat pair index


def _tiny(seed=4, E=4, H=256, I=128, T=8):
    gen = torch.Generator().manual_seed(seed)
    w = moe.moe_make_weights(E, H, I, gen)
    x, logits = moe.moe_make_inputs(T, H, E, gen)
    return x, logits, w


def test_layer_against_float64_dense():
    x, logits, (w13_q, w13_s, w2_q, w2_s) = _tiny()
    out, mid = moe.moe_forward(x, logits, w13_q, w13_s, w2_q, w2_s, top_k=2, out_dtype=torch.float32,
                               return_intermediates=True)
    ids, wts = mid['ids'], mid['weights'].double()
    xd = moe.dequantize_groups(mid['x_q'], mid['x_s']).double()
    want = torch.zeros(8, 256, dtype=torch.float64)
    for t in range(8):
        for k in range(2):
            e = ids[t, k].item()
            gu = moe.dequantize_blocks(w13_q[e], w13_s[e]).double() @ xd[t]
            h = gu[:128] / (1 + torch.exp(-gu[:128])) * gu[128:]
            hq, hs = moe.quantize_groups(h.float()[None])
            want[t] += wts[t, k] * (moe.dequantize_blocks(w2_q[e], w2_s[e]).double()
                                    @ moe.dequantize_groups(hq, hs)[0].double())
    assert moe.rel_rms_error(out, want) < 1e-4


def test_exact_integer_case():
    # scales 1, small-integer codes, zero logits except the winners: every partial sum is an
    # exactly representable integer, so fp32 evaluation order cannot matter.
    E, H, I, T = 2, 128, 128, 4
    gen = torch.Generator().manual_seed(5)
    w13 = torch.randint(-2, 3, (E, 2 * I, H), generator=gen).float()
    w2 = torch.randint(-2, 3, (E, H, I), generator=gen).float()
    x = torch.randint(-3, 4, (T, H), generator=gen).float()
    x[:, 0] = 448.0                                     # amax 448 -> activation scale exactly 1
    xq, xs = moe.quantize_groups(x)
    assert torch.all(xs == 1.0) and torch.equal(xq.float(), x)
    gu = x @ w13[0].T
    assert torch.equal(gu, (x.double() @ w13[0].double().T).float())


def test_single_expert_is_a_plain_mlp():
    x, logits, (w13_q, w13_s, w2_q, w2_s) = _tiny(6, E=1, T=5)
    out = moe.moe_forward(x, logits, w13_q, w13_s, w2_q, w2_s, top_k=1, out_dtype=torch.float32)
    xq, xs = moe.quantize_groups(x.float())
    gu = moe.dequantize_groups(xq, xs) @ moe.dequantize_blocks(w13_q[0], w13_s[0]).T
    h = moe.silu(gu[:, :128]) * gu[:, 128:]
    hq, hs = moe.quantize_groups(h)
    want = moe.dequantize_groups(hq, hs) @ moe.dequantize_blocks(w2_q[0], w2_s[0]).T
    torch.testing.assert_close(out, want, rtol=1e-6, atol=1e-6)


def test_block_scale_acts_on_its_k_slice_only():
    x, logits, (w13_q, w13_s, w2_q, w2_s) = _tiny(7, E=1, T=3)
    xq, xs = moe.quantize_groups(x.float())
    xd = moe.dequantize_groups(xq, xs)
    base = xd @ moe.dequantize_blocks(w13_q[0], w13_s[0]).T
    s2 = w13_s.clone()
    s2[0, 1, 0] *= 3.0                                  # rows 128..255, K columns 0..127
    bumped = xd @ moe.dequantize_blocks(w13_q[0], s2[0]).T
    delta = 2.0 * (xd[:, :128] @ moe.dequantize_blocks(w13_q[0], w13_s[0])[128:256, :128].T)
    torch.testing.assert_close(bumped[:, 128:256] - base[:, 128:256], delta, rtol=1e-4, atol=1e-4)
    assert torch.equal(bumped[:, :128], base[:, :128])


def test_silu_closed_form():
    v = torch.linspace(-20, 20, 101)
    torch.testing.assert_close(moe.silu(v), torch.nn.functional.silu(v), rtol=1e-6, atol=1e-7)
    assert moe.silu(torch.tensor(0.0)) == 0


def test_weight_generator_has_no_nan_codes():
    gen = torch.Generator().manual_seed(8)
    w13_q, w13_s, w2_q, w2_s = moe.moe_make_weights(2, 256, 128, gen)
    for q in (w13_q, w2_q, moe.random_e4m3((1000,), gen)):
        assert ((q.view(torch.uint8) & 0x7F) != 0x7F).all()
    assert (w13_s > 0.5 / 448 - 1e-9).all() and (w13_s < 1.5 / 448 + 1e-9).all()
    assert w13_s.shape == (2, 2, 2) and w2_s.shape == (2, 2, 1)


# ---- group-limited routing with a selection bias -------------------------------------------------

def _route_grouped_loops(logits, bias, top_k, n_group, topk_group, normalise, scale):
    T, E = logits.shape
    gs = E // n_group
    ids, weights = [], []
    for t in range(T):
        score = [float(torch.sigmoid(logits[t, e])) for e in range(E)]
        choice = [float(np.float32(score[e]) + np.float32(0.0 if bias is None else float(bias[e]))) for e in range(E)]
        value = []
        for g in range(n_group):
            best = sorted(choice[g * gs:(g + 1) * gs], reverse=True)[:2]
            value.append(float(np.float32(sum(np.float32(b) for b in best))))
        groups = sorted(range(n_group), key=lambda g: (-value[g], g))[:topk_group]
        candidates = [e for e in range(E) if e // gs in groups]
        chosen = sorted(candidates, key=lambda e: (-choice[e], e))[:top_k]
        w = np.array([score[e] for e in chosen], dtype=np.float32)
        if normalise:
            w = w / (w.sum(dtype=np.float32) + np.float32(1e-20))
        ids.append(chosen)
        weights.append(w * np.float32(scale))
    return np.array(ids), np.array(weights)


@pytest.mark.parametrize('shape', [(7, 16, 3, 4, 2, True, 1.0), (5, 64, 8, 8, 4, True, 2.5), (6, 32, 4, 4, 4, False, 1.0),
                                   (4, 24, 5, 3, 2, True, 0.5), (3, 8, 2, 8, 3, True, 1.0)])
def test_grouped_routing_matches_scalar_loops(shape):
    T, E, k, G, kg, norm, scale = shape
    gen = torch.Generator().manual_seed(T * 100 + E)
    logits = torch.randn(T, E, generator=gen)
    bias = 0.2 * torch.randn(E, generator=gen)
    ids, w, _ = moe.route_grouped(logits, bias, k, G, kg, norm, scale)
    want_ids, want_w = _route_grouped_loops(logits, bias, k, G, kg, norm, scale)
    np.testing.assert_array_equal(ids.numpy(), want_ids)
    np.testing.assert_allclose(w.numpy(), want_w, rtol=1e-6)


def test_grouped_routing_with_one_group_and_no_bias_is_plain_routing():
    gen = torch.Generator().manual_seed(21)
    logits = torch.randn(64, 256, generator=gen)
    ids, w, _ = moe.route_grouped(logits, None, 8, 1, 1)
    want_ids, want_w = moe.route(logits, 8)
    assert torch.equal(ids, want_ids)
    torch.testing.assert_close(w, want_w, rtol=1e-6, atol=0)


def test_grouped_routing_invariants():
    gen = torch.Generator().manual_seed(22)
    T, E, k, G, kg = 200, 256, 8, 8, 4
    logits = torch.randn(T, E, generator=gen)
    bias = 0.3 * torch.randn(E, generator=gen)
    ids, w, choice = moe.route_grouped(logits, bias, k, G, kg, True, 2.5)
    groups = ids // (E // G)
    assert all(len(set(row.tolist())) <= kg for row in groups)
    assert all(len(set(row.tolist())) == k for row in ids)
    torch.testing.assert_close(w.sum(dim=1), torch.full((T,), 2.5), rtol=1e-5, atol=0)
    # the bias moves the choice but not the weights: weights are ratios of unbiased sigmoids
    score = torch.sigmoid(logits).gather(1, ids.long())
    torch.testing.assert_close(w, 2.5 * score / score.sum(dim=1, keepdim=True), rtol=1e-5, atol=0)
    # a large bias on one expert of a group that stays forces that expert in
    big = bias.clone()
    big[5] = 10.0
    ids2, _, _ = moe.route_grouped(logits, big, k, G, kg)
    assert (ids2[:, 0] == 5).all()


def test_grouped_routing_matches_third_party_golden():
    from pathlib import Path
    z = np.load(Path(__file__).parent / 'golden' / 'router_golden.npz')
    for tag in 'abc':
        k, G, kg, norm = (int(v) for v in z[f'{tag}_params'])
        logits = torch.from_numpy(z[f'{tag}_logits'])
        # the fixture's logits are the fp32 product of its hidden states and router weight
        want_logits = torch.from_numpy(z[f'{tag}_hidden']) @ torch.from_numpy(z[f'{tag}_weight']).T
        torch.testing.assert_close(logits, want_logits, rtol=1e-4, atol=1e-5)
        ids, w, _ = moe.route_grouped(logits, torch.from_numpy(z[f'{tag}_bias']), k, G, kg, bool(norm),
                                      float(z[f'{tag}_scale'][0]))
        order = ids.argsort(dim=-1)
        np.testing.assert_array_equal(ids.gather(1, order).numpy(), z[f'{tag}_ids'])
        np.testing.assert_allclose(w.gather(1, order).numpy(), z[f'{tag}_weights'], rtol=1e-5)


def test_shared_expert_against_float64_dense():
    x, logits, (w13_q, w13_s, w2_q, w2_s) = _tiny()
    gen = torch.Generator().manual_seed(91)
    (sw13_q, sw13_s, sw2_q, sw2_s) = (t[0] for t in moe.moe_make_weights(1, 256, 256, generator=gen))
    out = moe.moe_forward_shared(x, logits, w13_q, w13_s, w2_q, w2_s, sw13_q, sw13_s, sw2_q, sw2_s, top_k=2,
                                 out_dtype=torch.float32)
    routed = moe.moe_forward(x, logits, w13_q, w13_s, w2_q, w2_s, top_k=2, out_dtype=torch.float32)
    xq, xs = moe.quantize_groups(x.float())
    xd = moe.dequantize_groups(xq, xs).double()
    want = routed.double()
    for t in range(x.shape[0]):
        gu = moe.dequantize_blocks(sw13_q, sw13_s).double() @ xd[t]
        h = gu[:256] / (1 + torch.exp(-gu[:256])) * gu[256:]
        hq, hs = moe.quantize_groups(h.float()[None])
        want[t] += moe.dequantize_blocks(sw2_q, sw2_s).double() @ moe.dequantize_groups(hq, hs)[0].double()
    assert moe.rel_rms_error(out, want) < 1e-4
    assert moe.rel_rms_error(out, routed) > 0.1       # the shared term is not negligible in this check


def test_router_logits_against_float64_and_golden():
    from pathlib import Path
    gen = torch.Generator().manual_seed(23)
    x = torch.randn(20, 192, generator=gen).bfloat16()
    w = torch.randn(48, 192, generator=gen)
    got = moe.router_logits(x, w)
    want = x.double() @ w.double().T
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)
    z = np.load(Path(__file__).parent / 'golden' / 'router_golden.npz')
    for tag in 'abc':
        got = moe.router_logits(torch.from_numpy(z[f'{tag}_hidden']).bfloat16(), torch.from_numpy(z[f'{tag}_weight']))
        torch.testing.assert_close(got, torch.from_numpy(z[f'{tag}_logits']), rtol=1e-5, atol=1e-6)


# ---- power-of-two (UE8M0) scales -----------------------------------------------------------------

def test_pow2_ceil_is_exact():
    gen = torch.Generator().manual_seed(61)
    v = torch.exp(torch.randn(4000, generator=gen) * 8).float()
    want = torch.pow(2.0, torch.ceil(torch.log2(v.double())))
    assert torch.equal(moe.pow2_ceil(v).double(), want)
    p = torch.ldexp(torch.ones(60), torch.arange(-30, 30))
    assert torch.equal(moe.pow2_ceil(p), p)
    assert torch.equal(moe.pow2_ceil(torch.nextafter(p, torch.full_like(p, float('inf')))), 2 * p)
    assert torch.equal(moe.pow2_ceil(torch.nextafter(p, torch.zeros_like(p))), p)


def test_pow2_group_quantisation_properties():
    gen = torch.Generator().manual_seed(62)
    v = torch.randn(64, 512, generator=gen) * torch.exp(torch.randn(64, 1, generator=gen) * 3)
    v[3, :128] = 0.0                                   # an all-zero group takes the floor
    v[4, 5] = 448.0 * 2 ** -3                          # amax/448 exactly a power of two
    v[4, :128] = v[4, :128].clamp(-56.0, 56.0)
    v[5, 130] = float(torch.nextafter(torch.tensor(448.0 * 4), torch.tensor(1e9)))   # just above
    v[5, 128:256] = v[5, 128:256].clamp(-1793.0, 1793.0)
    q, s = moe.quantize_groups(v, pow2=True)
    assert torch.equal(s, moe.pow2_ceil(s))                                  # powers of two
    amax = v.reshape(64, 4, 128).abs().amax(dim=-1).clamp_min(moe.AMAX_FLOOR).double()
    assert (s.double() * 448 >= amax).all() and (s.double() * 224 < amax).all()
    assert s[4, 0] == 2 ** -3 and s[5, 1] == 8.0
    # the division is exact, so the codes are the e4m3 rounding of v / s computed in float64
    want = (v.double().reshape(64, 4, 128) / s.double()[:, :, None]).float().to(torch.float8_e4m3fn)
    assert torch.equal(q.view(torch.uint8), want.reshape(64, 512).view(torch.uint8))
    top = q.float().reshape(64, 4, 128).abs().amax(dim=-1)
    live = amax > moe.AMAX_FLOOR
    assert (top[live] >= 224).all() and (top <= 448).all()      # amax/s in (224, 448] rounds to a code >= 224
    # idempotent on its own output
    dq = moe.dequantize_groups(q, s)
    q2, _ = moe.quantize_groups(dq, pow2=True)
    assert torch.equal(moe.dequantize_groups(q2, moe.quantize_groups(dq, pow2=True)[1]), dq)


def test_pow2_layer_against_float64_dense():
    gen = torch.Generator().manual_seed(63)
    w13_q, w13_s, w2_q, w2_s = moe.moe_make_weights(4, 256, 128, gen, pow2_scales=True)
    x, logits = moe.moe_make_inputs(8, 256, 4, gen)
    out, mid = moe.moe_forward(x, logits, w13_q, w13_s, w2_q, w2_s, top_k=2, out_dtype=torch.float32,
                               return_intermediates=True, pow2_scales=True)
    assert torch.equal(mid['x_s'], moe.pow2_ceil(mid['x_s'])) and torch.equal(mid['h_s'], moe.pow2_ceil(mid['h_s']))
    ids, wts = mid['ids'], mid['weights'].double()
    xd = moe.dequantize_groups(mid['x_q'], mid['x_s']).double()
    want = torch.zeros(8, 256, dtype=torch.float64)
    for t in range(8):
        for k in range(2):
            e = ids[t, k].item()
            gu = moe.dequantize_blocks(w13_q[e], w13_s[e]).double() @ xd[t]
            h = gu[:128] / (1 + torch.exp(-gu[:128])) * gu[128:]
            hq, hs = moe.quantize_groups(h.float()[None], pow2=True)
            want[t] += wts[t, k] * (moe.dequantize_blocks(w2_q[e], w2_s[e]).double()
                                    @ moe.dequantize_groups(hq, hs)[0].double())
    assert moe.rel_rms_error(out, want) < 1e-4
    with pytest.raises(AssertionError):
        moe.moe_forward(x, logits, w13_q, w13_s * 1.5, w2_q, w2_s, top_k=2, pow2_scales=True)


# ---- the bf16 RMS norm in front of the layer -----------------------------------------------------

def test_rmsnorm_bf16_closed_form_and_golden():
    from pathlib import Path
    gen = torch.Generator().manual_seed(71)
    x = (torch.randn(9, 384, generator=gen) * 3).bfloat16()
    w = (1.0 + 0.2 * torch.randn(384, generator=gen)).bfloat16()
    y = moe.rmsnorm_bf16(x, w)
    assert y.dtype == torch.bfloat16
    xd = x.double()
    want = w.double() * xd / torch.sqrt(xd.pow(2).mean(-1, keepdim=True) + 1e-6)
    assert ((y.double() - want).abs() <= want.abs() * 2.0 ** -7 + 1e-30).all()      # two bf16 roundings
    z = np.load(Path(__file__).parent / 'golden' / 'rmsnorm_golden.npz')
    got = moe.rmsnorm_bf16(torch.from_numpy(z['x']).bfloat16(), torch.from_numpy(z['weight']).bfloat16())
    want = torch.from_numpy(z['y'])
    # the module uses rsqrt, this restatement 1/sqrt: an fp32 ulp of the factor can move a value across a bf16 boundary
    assert (got.float() == want).float().mean() >= 0.995
    assert ((got.float() - want).abs() <= want.abs() * 2.0 ** -7).all()


def test_split_bf16x3_is_exact():
    gen = torch.Generator().manual_seed(77)
    w = torch.randn(50, 64, generator=gen) * torch.exp(4 * torch.randn(50, 1, generator=gen))
    w[0, :5] = torch.tensor([0.0, -0.0, 1e-30, 3e38, 2.0 ** -120])
    planes = moe.split_bf16x3(w)
    assert planes.dtype == torch.bfloat16 and planes.shape == (3, 50, 64)
    assert torch.equal((planes[0].float() + planes[1].float()) + planes[2].float(), w)
    assert torch.equal(planes.double().sum(0), w.double())
    # the first plane is w with its lower 16 bits cleared; the planes shrink by 2^-8 each
    assert torch.equal(planes[0].float().view(torch.int32), w.view(torch.int32) & -65536)
    assert (planes[1].float().abs() <= planes[0].float().abs() * 2.0 ** -7 + 1e-45).all()
    assert (planes[2].float().abs() <= planes[0].float().abs() * 2.0 ** -15 + 1e-45).all()
    # so a bf16 x times the planes gives the fp32 product terms exactly
    x = torch.randn(64, generator=gen).bfloat16()
    exact = (x.double()[None, :] * w.double()).sum(dim=1)
    via_planes = sum((x.double()[None, :] * planes[i].double()).sum(dim=1) for i in range(3))
    torch.testing.assert_close(via_planes, exact, rtol=1e-14, atol=0)
