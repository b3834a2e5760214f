"""GPU parity of the single-token causal convolution update against the oracle, through the C ABI.

The state is only moved, so it must be bit-exact. The output is fp32 arithmetic over at most 4 taps:
fp32 storage is held to rtol 1e-5; bf16 storage must be the oracle's bf16 value or its neighbour (the
kernel's fused multiply-adds and hardware exponential can put an fp32 result on the other side of a
bf16 rounding boundary), and at least 99 % of the outputs must be identical."""
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import gdn

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).parent / 'golden' / 'conv1d_update_golden.npz'


def run_kernel(capi, dev, x, state, weight, bias, key_dim, activation='silu'):
    B, C, _ = state.shape
    value_dim = C - 2 * key_dim
    dt = state.dtype
    state_d = state.to(dev).clone()
    v = torch.full((B, value_dim), float('nan'), dtype=dt, device=dev)
    q = k = None
    if key_dim:
        q = torch.full((B, key_dim), float('nan'), dtype=dt, device=dev)
        k = torch.full((B, key_dim), float('nan'), dtype=dt, device=dev)
    capi.causal_conv1d_update_launch(q, k, v, state_d, x.to(dev), weight.to(dev),
                                     None if bias is None else bias.to(dev), activation)
    torch.cuda.synchronize()
    out = torch.cat([q, k, v], dim=1) if key_dim else v
    return out.cpu(), state_d.cpu()


def assert_out_close(out, want):
    assert torch.isfinite(out.float()).all()
    if out.dtype == torch.float32:
        torch.testing.assert_close(out, want, rtol=1e-5, atol=1e-6)
        return
    a, b = out.float(), want.float()
    ulp = torch.maximum(a.abs(), b.abs()) * 2.0 ** -7            # one bf16 step at that magnitude, at most
    assert ((a - b).abs() <= ulp + 1e-30).all()
    assert (out == want).float().mean() >= 0.99


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('L,K', [(4, 4), (3, 4), (3, 3), (2, 3), (2, 2), (1, 2)])
@pytest.mark.parametrize('activation', ['silu', None])
def test_matches_oracle(capi, dev, dtype, L, K, activation):
    gen = torch.Generator().manual_seed(100 * L + K)
    for B, key_dim, value_dim, with_bias in ((3, 64, 128, True), (2, 8, 8, False), (5, 2048 + 8, 4096 + 24, True),
                                             (1, 0, 40, True)):
        x, state, weight, bias = gdn.conv_make_inputs(B, key_dim, value_dim, L, K, dtype, generator=gen)
        if not with_bias:
            bias = None
        want_state = state.clone()
        want = gdn.causal_conv1d_update(x, want_state, weight, bias, activation)
        out, new_state = run_kernel(capi, dev, x, state, weight, bias, key_dim, activation)
        assert torch.equal(new_state, want_state)
        assert_out_close(out, want)


def test_golden_fixture(capi, dev):
    z = np.load(GOLDEN)
    for tag in 'abc':
        state = torch.from_numpy(z[f'{tag}_state0'])
        weight = torch.from_numpy(z[f'{tag}_weight'])
        bias = torch.from_numpy(z[f'{tag}_bias']) if z[f'{tag}_bias'].size else None
        for t in range(3):
            out, state = run_kernel(capi, dev, torch.from_numpy(z[f'{tag}_x{t}']), state, weight, bias, 8)
            np.testing.assert_allclose(out.numpy(), z[f'{tag}_out{t}'], rtol=1e-5, atol=1e-6)
            np.testing.assert_array_equal(state.numpy(), z[f'{tag}_state{t + 1}'])


def test_token_by_token_equals_one_causal_convolution(capi, dev):
    gen = torch.Generator().manual_seed(8)
    C, K, T = 64, 4, 7
    xs = torch.randn(2, C, T, generator=gen)
    weight = torch.randn(C, K, generator=gen)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(xs, (K - 1, 0)), weight[:, None, :], groups=C)
    state = torch.zeros(2, C, K - 1)
    outs = []
    for t in range(T):
        out, state = run_kernel(capi, dev, xs[:, :, t].contiguous(), state, weight, None, 16, None)
        outs.append(out)
    torch.testing.assert_close(torch.stack(outs, dim=2), want, rtol=1e-5, atol=1e-6)
    assert torch.equal(state, xs[:, :, T - (K - 1):])


def test_layer_decode_chain_at_the_workload_shape(capi, dev):
    # convolution update -> fused GDN step (q/k normalisation and gates inside), B=256, 16/32 heads of 128:
    # what a layer runs per token, against the oracle's chain of the same two steps
    gen = torch.Generator().manual_seed(9)
    B, Hv, Hqk, d = 256, 32, 16, 128
    x, cstate, weight, bias = gdn.conv_make_inputs(B, Hqk * d, Hv * d, 4, 4, torch.bfloat16, generator=gen)
    _, _, _, a, b, a_log, dt_bias, state = gdn.gdn_make_raw_inputs(B, Hv, Hqk, qkv_dtype=torch.bfloat16,
                                                                   generator=gen)
    want_cstate = cstate.clone()
    mixed = gdn.causal_conv1d_update(x, want_cstate, weight, bias)
    q_w, k_w, v_w = (t.reshape(B, -1, d) for t in mixed.split([Hqk * d, Hqk * d, Hv * d], dim=1))

    x, cstate, weight, bias, a, b, a_log, dt_bias = (t.to(dev) for t in (x, cstate, weight, bias, a, b, a_log,
                                                                         dt_bias))
    q = torch.empty(B, Hqk * d, dtype=torch.bfloat16, device=dev)
    k = torch.empty_like(q)
    v = torch.empty(B, Hv * d, dtype=torch.bfloat16, device=dev)
    capi.causal_conv1d_update_launch(q, k, v, cstate, x, weight, bias)
    s = state.to(dev)
    o = torch.empty(B, Hv, d, dtype=torch.float32, device=dev)
    capi.gdn_decode_fused_launch(o, s, q.view(B, Hqk, d), k.view(B, Hqk, d), v.view(B, Hv, d), a, b, a_log,
                                 dt_bias)
    torch.cuda.synchronize()
    assert torch.equal(cstate.cpu(), want_cstate)
    assert_out_close(torch.cat([q, k, v], dim=1).cpu(), mixed)
    # the recurrence is compared on the kernel's own q, k, v (a neighbouring bf16 value of one input moves
    # the state update by more than the recurrence's own 1e-3 bound)
    want_o, want_s = gdn.gdn_decode_fused_step(q.view(B, Hqk, d).cpu(), k.view(B, Hqk, d).cpu(),
                                               v.view(B, Hv, d).cpu(), a.cpu(), b.cpu(), a_log.cpu(),
                                               dt_bias.cpu(), state.clone())
    assert gdn.gdn_close(o.cpu(), want_o) and gdn.gdn_close(s.cpu(), want_s)
    assert q_w.shape == (B, Hqk, d) and k_w.shape == (B, Hqk, d) and v_w.shape == (B, Hv, d)


def test_rejects_unsupported_shapes(capi, dev):
    def tensors(key_dim, value_dim, L, K):
        C = 2 * key_dim + value_dim
        z = lambda *s: torch.zeros(*s, device=dev)
        return z(1, key_dim), z(1, key_dim), z(1, value_dim), z(1, C, L), z(1, C), z(C, K)

    for shape in ((12, 8, 3, 4), (8, 8, 5, 4), (8, 8, 2, 4), (8, 8, 4, 5)):
        with pytest.raises(capi.LaunchRejected):
            capi.causal_conv1d_update_launch(*tensors(*shape))
    q, k, v, state, x, w = tensors(8, 8, 4, 4)
    with pytest.raises(capi.LaunchRejected):
        capi.causal_conv1d_update_launch(q, k, v, state, torch.zeros(25, device=dev)[1:].view(1, 24), w)   # misaligned x
    torch.cuda.synchronize()
