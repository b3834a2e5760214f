"""Group-limited, bias-corrected routing on the GPU against the oracle, through the C ABI.

Bar: expert ids bit-exact, in the oracle's order (descending choice value, ties to the lower id). The kernel's
sigmoid and the oracle's may round differently in the last place, so a token whose decision hangs on two choice
values (or two group values) a few ulp apart may differ; such tokens are counted and must stay below 1 in 1000
(none occurs at the seeds used here up to 1000 tokens). Weights: rtol 1e-5."""
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import moe

pytestmark = pytest.mark.gpu


def run_kernel(capi, dev, logits, bias, k, G, kg, norm=True, scale=1.0):
    T = logits.shape[0]
    ids = torch.full((T, k), -1, dtype=torch.int32, device=dev)
    w = torch.full((T, k), float('nan'), device=dev)
    capi.moe_route_grouped_launch(ids, w, logits.to(dev), None if bias is None else bias.to(dev), G, kg, norm, scale)
    torch.cuda.synchronize()
    return ids.cpu(), w.cpu()


def check(capi, dev, logits, bias, k, G, kg, norm=True, scale=1.0):
    want_ids, want_w, choice = moe.route_grouped(logits, bias, k, G, kg, norm, scale)
    ids, w = run_kernel(capi, dev, logits, bias, k, G, kg, norm, scale)
    same = (ids == want_ids).all(dim=1)
    close_calls = 0
    for t in torch.nonzero(~same).flatten().tolist():
        assert len(set(ids[t].tolist())) == k
        a, b = set(ids[t].tolist()), set(want_ids[t].tolist())
        if a == b:      # same experts in another order: two of them must tie within a few ulp
            vals = choice[t][ids[t].long()].sort().values
            assert (vals[1:] - vals[:-1]).min() <= 4 * 2.0 ** -23 * vals.abs().max().clamp_min(1.0)
        close_calls += 1
    assert close_calls <= max(1, logits.shape[0] // 1000), close_calls
    torch.testing.assert_close(w[same], want_w[same], rtol=1e-5, atol=1e-9)
    return ids, w


@pytest.mark.parametrize('shape', [(64, 256, 8, 8, 4), (1000, 256, 8, 8, 4), (37, 64, 6, 4, 2), (5, 32, 4, 1, 1),
                                   (130, 512, 8, 16, 5), (9, 8, 2, 8, 3), (64, 384, 8, 8, 4), (3, 24, 5, 3, 2)])
@pytest.mark.parametrize('norm,scale', [(True, 2.5), (False, 1.0)])
def test_matches_oracle(capi, dev, shape, norm, scale):
    T, E, k, G, kg = shape
    gen = torch.Generator().manual_seed(T + E)
    logits = torch.randn(T, E, generator=gen)
    bias = 0.2 * torch.randn(E, generator=gen)
    check(capi, dev, logits, bias, k, G, kg, norm, scale)
    check(capi, dev, logits, None, k, G, kg, norm, scale)


def test_prefill_size_and_biased_experts(capi, dev):
    gen = torch.Generator().manual_seed(77)
    logits = torch.randn(8192, 256, generator=gen)
    logits[:, torch.randperm(256, generator=gen)[:16]] += 2.0
    bias = 0.1 * torch.randn(256, generator=gen)
    ids, w = check(capi, dev, logits, bias, 8, 8, 4, True, 2.5)
    assert all(len(set(r.tolist())) <= 4 for r in (ids[:500] // 32))
    torch.testing.assert_close(w.sum(dim=1), torch.full((8192,), 2.5), rtol=1e-5, atol=0)


def test_one_group_without_bias_is_the_plain_router(capi, dev):
    gen = torch.Generator().manual_seed(78)
    logits = torch.randn(300, 256, generator=gen).to(dev)
    ids = torch.empty(300, 8, dtype=torch.int32, device=dev)
    w = torch.empty(300, 8, device=dev)
    capi.moe_route_launch(ids, w, logits)
    ids2, w2 = run_kernel(capi, dev, logits.cpu(), None, 8, 1, 1)
    torch.cuda.synchronize()
    assert torch.equal(ids.cpu(), ids2)
    torch.testing.assert_close(w.cpu(), w2, rtol=1e-6, atol=0)


def test_ties_go_to_the_lower_group_and_the_lower_expert(capi, dev):
    logits = torch.zeros(4, 64)
    ids, w = run_kernel(capi, dev, logits, None, 6, 8, 2)
    assert torch.equal(ids, torch.tensor([[0, 1, 2, 3, 4, 5]] * 4, dtype=torch.int32))
    torch.testing.assert_close(w, torch.full((4, 6), 1 / 6), rtol=1e-6, atol=0)
    logits[:, 40:48] = 1.0          # group 5 now wins, group 0 is second
    ids, _ = run_kernel(capi, dev, logits, None, 6, 8, 2)
    assert torch.equal(ids, torch.tensor([[40, 41, 42, 43, 44, 45]] * 4, dtype=torch.int32))
    ids, _ = run_kernel(capi, dev, logits, None, 10, 8, 2)
    assert torch.equal(ids[0], torch.tensor([40, 41, 42, 43, 44, 45, 46, 47, 0, 1], dtype=torch.int32))


def test_third_party_golden_fixture(capi, dev):
    z = np.load(Path(__file__).parent / 'golden' / 'router_golden.npz')
    for tag in 'abc':
        k, G, kg, norm = (int(v) for v in z[f'{tag}_params'])
        ids, w = run_kernel(capi, dev, torch.from_numpy(z[f'{tag}_logits']), torch.from_numpy(z[f'{tag}_bias']),
                            k, G, kg, bool(norm), float(z[f'{tag}_scale'][0]))
        order = ids.argsort(dim=-1)
        np.testing.assert_array_equal(ids.gather(1, order).numpy(), z[f'{tag}_ids'])
        np.testing.assert_allclose(w.gather(1, order).numpy(), z[f'{tag}_weights'], rtol=1e-5)


def test_rejects_unsupported_shapes(capi, dev):
    logits = torch.zeros(2, 256, device=dev)
    ids = torch.zeros(2, 8, dtype=torch.int32, device=dev)
    w = torch.zeros(2, 8, device=dev)
    for G, kg in ((7, 2), (8, 9), (128, 4), (8, 0)):
        with pytest.raises(capi.LaunchRejected):
            capi.moe_route_grouped_launch(ids, w, logits, None, G, kg)
    ids = torch.zeros(2, 40, dtype=torch.int32, device=dev)    # 40 experts wanted, 32 stay
    w = torch.zeros(2, 40, device=dev)
    with pytest.raises(capi.LaunchRejected):
        capi.moe_route_grouped_launch(ids, w, logits, None, 8, 1)
    torch.cuda.synchronize()


# ---- router projection ---------------------------------------------------------------------------

def run_logits(capi, dev, x, w):
    T, H = x.shape
    E = w.shape[0]
    logits = torch.full((T, E), float('nan'), device=dev)
    nbytes = capi.moe_router_logits_workspace_bytes(T, H, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev) if nbytes else None
    capi.moe_router_logits_launch(logits, x.to(dev), w.to(dev), ws)
    torch.cuda.synchronize()
    return logits.cpu()


def logits_bound(x, w):
    # fp32 accumulation of H products in any order: |err| <= H * 2^-24 * sum |x_h w_eh| (loose by sqrt(H))
    return x.shape[1] * 2.0 ** -24 * (x.double().abs() @ w.double().abs().T)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('shape', [(64, 7168, 256), (1, 64, 32), (100, 448, 72), (700, 1024, 256), (33, 128, 1),
                                   (130, 2048, 384)])
def test_router_logits_match_float64(capi, dev, shape, dtype):
    T, H, E = shape
    gen = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, H, generator=gen).to(dtype)
    w = torch.randn(E, H, generator=gen) * H ** -0.5
    got = run_logits(capi, dev, x, w)
    want = x.double() @ w.double().T
    assert torch.isfinite(got).all()
    assert ((got.double() - want).abs() <= logits_bound(x, w)).all()
    # as close to the exact product as the oracle's own fp32 evaluation
    err = (got.double() - want).abs().max().item()
    ref_err = (moe.router_logits(x, w).double() - want).abs().max().item()
    assert err <= 4 * ref_err + 1e-7


def test_router_logits_exact_on_integers(capi, dev):
    # small integers: every partial sum is an exact fp32 integer, so any summation order gives the same bits
    gen = torch.Generator().manual_seed(51)
    x = torch.randint(-8, 9, (96, 512), generator=gen).float().bfloat16()
    w = torch.randint(-8, 9, (64, 512), generator=gen).float()
    assert torch.equal(run_logits(capi, dev, x, w), x.float() @ w.T)


def test_router_logits_golden_fixture(capi, dev):
    z = np.load(Path(__file__).parent / 'golden' / 'router_golden.npz')
    for tag in 'a':                       # (the other two cases have hidden = 32, below the kernel's 64 grain)
        got = run_logits(capi, dev, torch.from_numpy(z[f'{tag}_hidden']).bfloat16(), torch.from_numpy(z[f'{tag}_weight']))
        torch.testing.assert_close(got, torch.from_numpy(z[f'{tag}_logits']), rtol=1e-5, atol=1e-6)


def test_projection_then_grouped_routing_at_prefill_size(capi, dev):
    # hidden states -> logits -> experts, against the oracle's chain; a token may differ only on a near-tie
    gen = torch.Generator().manual_seed(52)
    T, H, E = 8192, 1024, 256
    x = torch.randn(T, H, generator=gen).bfloat16()
    w = torch.randn(E, H, generator=gen) * H ** -0.5
    bias = 0.1 * torch.randn(E, generator=gen)
    logits = run_logits(capi, dev, x, w)
    ids, _ = run_kernel(capi, dev, logits, bias, 8, 8, 4, True, 2.5)
    want_ids, _, _ = moe.route_grouped(moe.router_logits(x, w), bias, 8, 8, 4, True, 2.5)
    differing = (ids != want_ids).any(dim=1).sum().item()
    assert differing <= 8, differing        # logits differ in the last place: 1 token in 1000 may flip


# ---- router projection with the weight split into three bf16 planes -------------------------------------------

def run_logits_split(capi, dev, x, w):
    T, H = x.shape
    E = w.shape[0]
    planes = torch.empty(3, E, H, dtype=torch.bfloat16, device=dev)
    capi.moe_router_split_weight_launch(planes, w.to(dev))
    logits = torch.full((T, E), float('nan'), device=dev)
    nbytes = capi.moe_router_logits_workspace_bytes(T, H, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev) if nbytes else None
    capi.moe_router_logits_split_launch(logits, x.to(dev), planes, ws)
    torch.cuda.synchronize()
    return logits.cpu(), planes.cpu()


@pytest.mark.parametrize('shape', [(64, 7168, 256), (1, 64, 32), (100, 448, 72), (700, 1024, 256), (33, 128, 1),
                                   (130, 2048, 384), (6200, 448, 250), (12345, 64, 70)])   # the last two: workgroup-tiled kernel
def test_split_weight_logits_match_float64(capi, dev, shape):
    T, H, E = shape
    gen = torch.Generator().manual_seed(T + E + 1)
    x = torch.randn(T, H, generator=gen).bfloat16()
    w = torch.randn(E, H, generator=gen) * H ** -0.5
    w[0, :4] = torch.tensor([0.0, 1e-30, -3e38, 2.0 ** -120])
    got, planes = run_logits_split(capi, dev, x, w)
    # the planes are the oracle's, and their sum is the weight, bit for bit
    assert torch.equal(planes.view(torch.int16), moe.split_bf16x3(w).view(torch.int16))
    assert torch.equal((planes[0].float() + planes[1].float()) + planes[2].float(), w)
    w[0, 2] = 0.0                                  # (keep the reference finite)
    got, _ = run_logits_split(capi, dev, x, w)
    want = x.double() @ w.double().T
    assert torch.isfinite(got).all()
    assert ((got.double() - want).abs() <= logits_bound(x, w)).all()
    err = (got.double() - want).abs().max().item()
    ref_err = (moe.router_logits(x, w).double() - want).abs().max().item()
    assert err <= 4 * ref_err + 1e-7


def test_split_weight_logits_exact_on_integers_and_routing_chain(capi, dev):
    gen = torch.Generator().manual_seed(53)
    x = torch.randint(-8, 9, (96, 512), generator=gen).float().bfloat16()
    w = torch.randint(-8, 9, (64, 512), generator=gen).float()
    got, _ = run_logits_split(capi, dev, x, w)
    assert torch.equal(got, x.float() @ w.T)
    # hidden states -> logits -> experts at prefill size, against the oracle's chain
    T, H, E = 8192, 1024, 256
    x = torch.randn(T, H, generator=gen).bfloat16()
    w = torch.randn(E, H, generator=gen) * H ** -0.5
    bias = 0.1 * torch.randn(E, generator=gen)
    logits, _ = run_logits_split(capi, dev, x, w)
    ids, _ = run_kernel(capi, dev, logits, bias, 8, 8, 4, True, 2.5)
    want_ids, _, _ = moe.route_grouped(moe.router_logits(x, w), bias, 8, 8, 4, True, 2.5)
    assert (ids != want_ids).any(dim=1).sum().item() <= 8


def test_router_logits_rejects_bad_arguments(capi, dev):
    logits = torch.zeros(4, 32, device=dev)
    w = torch.zeros(32, 96, device=dev)
    with pytest.raises(capi.LaunchRejected):          # hidden not a multiple of 64
        capi.moe_router_logits_launch(logits, torch.zeros(4, 96, device=dev), w)
    w = torch.zeros(32, 7168, device=dev)
    with pytest.raises(capi.LaunchRejected):          # K is split for 4 tokens: scratch needed
        capi.moe_router_logits_launch(logits, torch.zeros(4, 7168, device=dev), w)
    torch.cuda.synchronize()


# ---- RMS norm fused with the activation quantiser -------------------------------------------------

@pytest.mark.parametrize('shape', [(64, 7168), (5, 128), (300, 2048), (1, 8192), (33, 384)])
@pytest.mark.parametrize('config', [0, 32])
def test_rmsnorm_quant(capi, dev, shape, config):
    R, C = shape
    gen = torch.Generator().manual_seed(R + C)
    x = (torch.randn(R, C, generator=gen) * torch.exp(torch.randn(R, 1, generator=gen))).bfloat16()
    w = (1.0 + 0.2 * torch.randn(C, generator=gen)).bfloat16()
    q = torch.empty(R, C, dtype=torch.uint8, device=dev)
    s = torch.empty(R, C // 128, device=dev)
    y = torch.empty(R, C, dtype=torch.bfloat16, device=dev)
    capi.moe_rmsnorm_quant_launch(q, s, y, x.to(dev), w.to(dev), 1e-6, config)
    torch.cuda.synchronize()
    # the normalised row: the oracle's bf16 value, or its neighbour where the fp32 sums of squares differ in the
    # last place (different order of the additions) and the value sits on a bf16 rounding boundary
    want_y = moe.rmsnorm_bf16(x, w)
    assert (y.cpu() == want_y).float().mean().item() >= 0.995
    assert ((y.cpu().float() - want_y.float()).abs() <= want_y.float().abs() * 2.0 ** -7).all()
    # the quantisation of the kernel's own y: bit-exact
    want_q, want_s = moe.quantize_groups(y.cpu().float(), pow2=config == 32)
    assert torch.equal(s.cpu(), want_s)
    assert torch.equal(q.cpu(), want_q.view(torch.uint8))
    # y is optional
    q2 = torch.empty_like(q)
    s2 = torch.empty_like(s)
    capi.moe_rmsnorm_quant_launch(q2, s2, None, x.to(dev), w.to(dev), 1e-6, config)
    torch.cuda.synchronize()
    assert torch.equal(q2, q) and torch.equal(s2, s)


def test_rmsnorm_quant_golden_fixture(capi, dev):
    z = np.load(Path(__file__).parent / 'golden' / 'rmsnorm_golden.npz')
    x, w = torch.from_numpy(z['x']).bfloat16(), torch.from_numpy(z['weight']).bfloat16()
    R, C = x.shape
    q = torch.empty(R, C, dtype=torch.uint8, device=dev)
    s = torch.empty(R, C // 128, device=dev)
    y = torch.empty(R, C, dtype=torch.bfloat16, device=dev)
    capi.moe_rmsnorm_quant_launch(q, s, y, x.to(dev), w.to(dev))
    torch.cuda.synchronize()
    want = torch.from_numpy(z['y'])
    assert (y.cpu().float() == want).float().mean().item() >= 0.995
    assert ((y.cpu().float() - want).abs() <= want.abs() * 2.0 ** -7).all()


def test_rmsnorm_quant_rejects_bad_shapes(capi, dev):
    x = torch.zeros(2, 8320, dtype=torch.bfloat16, device=dev)        # more than 8192 columns
    with pytest.raises(capi.LaunchRejected):
        capi.moe_rmsnorm_quant_launch(torch.empty(2, 8320, dtype=torch.uint8, device=dev),
                                      torch.empty(2, 65, device=dev), None, x, torch.zeros(8320, dtype=torch.bfloat16, device=dev))
    torch.cuda.synchronize()
