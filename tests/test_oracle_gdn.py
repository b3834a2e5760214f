"""Pins the GDN decode oracle: brute force, invariants and a third-party golden fixture."""
import math
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import gdn

GOLDEN_DIR = Path(__file__).parent / 'golden'
GOLDEN = GOLDEN_DIR / 'gdn_decode_golden.npz'


def _tiny(seed=0, B=2, Hv=4, Hqk=2, dk=8, dv=4):
    gen = torch.Generator().manual_seed(seed)
    return gdn.gdn_make_inputs(B, Hv, Hqk, dk, dv, generator=gen)


def test_vectorised_step_matches_float64_loops():
    q, k, v, g, beta, state = _tiny()
    want_o, want_s = gdn.gdn_decode_loops_f64(*(t.numpy() for t in (q, k, v, g, beta, state)))
    o, s = gdn.gdn_decode_step(q, k, v, g, beta, state.clone())
    np.testing.assert_allclose(o.numpy(), want_o, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(s.numpy(), want_s, rtol=1e-5, atol=1e-7)


def test_state_is_updated_in_place_and_returned():
    q, k, v, g, beta, state = _tiny(1)
    before = state.clone()
    o, s = gdn.gdn_decode_step(q, k, v, g, beta, state)
    assert s.data_ptr() == state.data_ptr()
    assert not torch.equal(before, state)


def test_beta_zero_is_pure_decay():
    q, k, v, g, beta, state = _tiny(2)
    s0 = state.clone()
    o, s = gdn.gdn_decode_step(q, k, v, g, torch.zeros_like(beta), state)
    torch.testing.assert_close(s, s0 * g[:, :, None, None])
    rep = 2
    want_o = torch.einsum('bhij,bhi->bhj', s0, q.repeat_interleave(rep, 1)) * g[:, :, None] * 8 ** -0.5
    torch.testing.assert_close(o, want_o, rtol=1e-5, atol=1e-7)


def test_delta_rule_writes_v_under_key():
    # g = 1, beta = 1, |k| = 1: after the step the state returns v when probed with k.
    q, k, v, g, beta, state = _tiny(3)
    o, s = gdn.gdn_decode_step(q, k, v, torch.ones_like(g), torch.ones_like(beta), state)
    probe = torch.einsum('bhij,bhi->bhj', s, k.repeat_interleave(2, 1))
    torch.testing.assert_close(probe, v, rtol=1e-5, atol=1e-6)


def test_folded_single_pass_identity():
    # o = scale*(g*S0^T q + (k.q)*delta) with delta = beta*(v - g*S0^T k): the form the kernel uses
    q, k, v, g, beta, state = _tiny(4, dk=16, dv=8)
    s0 = state.double()
    qd, kd = q.double().repeat_interleave(2, 1), k.double().repeat_interleave(2, 1)
    a = torch.einsum('bhij,bhi->bhj', s0, kd)
    c = torch.einsum('bhij,bhi->bhj', s0, qd)
    gd, bd = g.double()[:, :, None], beta.double()[:, :, None]
    delta = bd * (v.double() - gd * a)
    want_o = 16 ** -0.5 * (gd * c + (kd * qd).sum(-1, keepdim=True) * delta)
    want_s = gd[..., None] * s0 + kd[..., None] * delta[:, :, None, :]
    o, s = gdn.gdn_decode_step(q, k, v, g, beta, state)
    torch.testing.assert_close(o.double(), want_o, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(s.double(), want_s, rtol=1e-5, atol=1e-7)


def test_gqa_equals_repeated_heads():
    q, k, v, g, beta, state = _tiny(5, Hv=6, Hqk=3)
    o1, s1 = gdn.gdn_decode_step(q, k, v, g, beta, state.clone())
    o2, s2 = gdn.gdn_decode_step(q.repeat_interleave(2, 1), k.repeat_interleave(2, 1), v, g, beta,
                                 state.clone())
    assert torch.equal(o1, o2) and torch.equal(s1, s2)


def test_linear_in_state_and_v():
    q, k, v, g, beta, state = _tiny(6)
    o1, s1 = gdn.gdn_decode_step(q, k, v, g, beta, state.clone())
    o2, s2 = gdn.gdn_decode_step(q, k, 3 * v, g, beta, 3 * state.clone())
    torch.testing.assert_close(o2, 3 * o1, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(s2, 3 * s1, rtol=1e-5, atol=1e-7)


def test_bf16_inputs_are_upcast():
    q, k, v, g, beta, state = _tiny(7)
    qb, kb, vb = q.bfloat16(), k.bfloat16(), v.bfloat16()
    o1, _ = gdn.gdn_decode_step(qb, kb, vb, g, beta, state.clone())
    o2, _ = gdn.gdn_decode_step(qb.float(), kb.float(), vb.float(), g, beta, state.clone())
    assert o1.dtype == torch.float32 and torch.equal(o1, o2)


def test_input_distribution():
    gen = torch.Generator().manual_seed(11)
    q, k, v, g, beta, state = gdn.gdn_make_inputs(8, 32, 16, generator=gen)
    torch.testing.assert_close(q.norm(dim=-1), torch.ones(8, 16), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(k.norm(dim=-1), torch.ones(8, 16), rtol=1e-5, atol=1e-5)
    assert (g > 0).all() and (g <= 1).all() and (beta > 0).all() and (beta < 1).all()
    assert abs(state.std().item() - 0.02) < 1e-3
    assert q.shape == (8, 16, 128) and v.shape == (8, 32, 128) and state.shape == (8, 32, 128, 128)


def test_golden_fixture_from_third_party_recurrence():
    z = np.load(GOLDEN)
    ins = [torch.from_numpy(z[n]) for n in ('q', 'k', 'v', 'g', 'beta', 'state')]
    o, s = gdn.gdn_decode_step(*ins[:5], ins[5].clone())
    np.testing.assert_allclose(o.numpy(), z['o'], rtol=2e-5, atol=1e-7)
    np.testing.assert_allclose(s.numpy(), z['new_state'], rtol=2e-5, atol=1e-7)


# ---- the caller's pre-step (L2 normalisation and gates) ------------------------------------------

FUSED_GOLDEN = Path(__file__).parent / 'golden' / 'gdn_fused_golden.npz'


def test_prestep_against_float64_closed_forms():
    gen = torch.Generator().manual_seed(21)
    qr, kr, v, a, b, a_log, dt_bias, _ = gdn.gdn_make_raw_inputs(3, 6, 3, 16, 8, generator=gen)
    qn, kn, g, beta = gdn.gdn_prestep(qr, kr, a, b, a_log, dt_bias)
    q64 = qr.double()
    want_q = q64 / torch.sqrt((q64 * q64).sum(-1, keepdim=True) + 1e-6)
    torch.testing.assert_close(qn.double(), want_q, rtol=1e-6, atol=1e-7)
    x = (a.double() + dt_bias.double())
    want_g = torch.exp(-torch.exp(a_log.double()) * torch.log1p(torch.exp(x)))   # softplus = log(1 + e^x)
    torch.testing.assert_close(g.double(), want_g, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(beta.double(), 1 / (1 + torch.exp(-b.double())), rtol=1e-6, atol=1e-7)
    assert (g > 0).all() and (g < 1).all()


def test_prestep_normalises_and_ignores_the_scale_of_q_and_k():
    gen = torch.Generator().manual_seed(22)
    qr, kr, v, a, b, a_log, dt_bias, state = gdn.gdn_make_raw_inputs(2, 4, 2, 32, 16, generator=gen)
    qn, kn, _, _ = gdn.gdn_prestep(qr, kr, a, b, a_log, dt_bias)
    torch.testing.assert_close(qn.norm(dim=-1), torch.ones(2, 2), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(kn.norm(dim=-1), torch.ones(2, 2), rtol=1e-5, atol=1e-5)
    o1, s1 = gdn.gdn_decode_fused_step(qr, kr, v, a, b, a_log, dt_bias, state.clone())
    o2, s2 = gdn.gdn_decode_fused_step(7.0 * qr, 0.25 * kr, v, a, b, a_log, dt_bias, state.clone())
    torch.testing.assert_close(o1, o2, rtol=1e-4, atol=1e-6)      # up to the 1e-6 under the root
    torch.testing.assert_close(s1, s2, rtol=1e-4, atol=1e-6)


def test_prestep_limits():
    gen = torch.Generator().manual_seed(23)
    qr, kr, v, a, b, a_log, dt_bias, state = gdn.gdn_make_raw_inputs(2, 4, 4, 16, 8, generator=gen)
    _, _, g, _ = gdn.gdn_prestep(qr, kr, a, b, torch.full_like(a_log, -60.0), dt_bias)
    assert torch.equal(g, torch.ones_like(g))                    # no decay
    _, _, _, beta = gdn.gdn_prestep(qr, kr, a, torch.full_like(b, -100.0), a_log, dt_bias)
    assert torch.equal(beta, torch.zeros_like(beta))             # nothing is written
    o, s = gdn.gdn_decode_fused_step(qr, kr, v, a, torch.full_like(b, -100.0), torch.full_like(a_log, -60.0),
                                     dt_bias, state.clone())
    assert torch.equal(s, state)


def test_fused_step_is_prestep_then_step():
    gen = torch.Generator().manual_seed(24)
    qr, kr, v, a, b, a_log, dt_bias, state = gdn.gdn_make_raw_inputs(2, 6, 3, 32, 16, generator=gen)
    qn, kn, g, beta = gdn.gdn_prestep(qr, kr, a, b, a_log, dt_bias)
    want_o, want_s = gdn.gdn_decode_loops_f64(qn, kn, v, g, beta, state)
    o, s = gdn.gdn_decode_fused_step(qr, kr, v, a, b, a_log, dt_bias, state.clone())
    np.testing.assert_allclose(o.numpy(), want_o, rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(s.numpy(), want_s, rtol=1e-4, atol=1e-6)


def test_fused_golden_fixture_from_third_party_layer_functions():
    z = np.load(FUSED_GOLDEN)
    ins = [torch.from_numpy(z[n]) for n in ('q', 'k', 'v', 'a', 'b', 'a_log', 'dt_bias', 'state')]
    o, s = gdn.gdn_decode_fused_step(*ins[:7], ins[7].clone())
    np.testing.assert_allclose(o.numpy(), z['o'], rtol=5e-5, atol=2e-7)
    np.testing.assert_allclose(s.numpy(), z['new_state'], rtol=5e-5, atol=2e-7)


# ---- single-token causal convolution update ----------------------------------------------------

def _conv_loops(x, state, weight, bias, activation):
    B, C, L = state.shape
    K = weight.shape[1]
    out = np.zeros((B, C))
    new_state = np.zeros((B, C, L))
    for b in range(B):
        for c in range(C):
            seq = [float(state[b, c, i]) for i in range(L)] + [float(x[b, c])]
            y = float(bias[c]) if bias is not None else 0.0
            for j in range(K):
                y += float(weight[c, j]) * seq[len(seq) - K + j]
            out[b, c] = y / (1.0 + math.exp(-y)) if activation == 'silu' else y
            new_state[b, c] = seq[1:]
    return out, new_state


@pytest.mark.parametrize('L,K', [(4, 4), (3, 4), (2, 2), (1, 2), (3, 3)])
@pytest.mark.parametrize('activation', ['silu', None])
def test_conv_update_matches_scalar_loops(L, K, activation):
    gen = torch.Generator().manual_seed(10 * L + K)
    x, state, weight, bias = gdn.conv_make_inputs(2, 8, 8, L, K, torch.float32, generator=gen)
    want_out, want_state = _conv_loops(x.numpy(), state.numpy(), weight.numpy(), bias.numpy(), activation)
    out = gdn.causal_conv1d_update(x, state, weight, bias, activation)
    np.testing.assert_allclose(out.numpy(), want_out, rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(state.numpy(), want_state.astype(np.float32))


def test_conv_update_is_the_library_convolution_of_the_concatenated_sequence():
    gen = torch.Generator().manual_seed(3)
    x, state, weight, bias = gdn.conv_make_inputs(3, 8, 16, 4, 4, torch.float32, generator=gen)
    seq = torch.cat([state, x[:, :, None]], dim=2)
    want = torch.nn.functional.conv1d(seq, weight[:, None, :], bias, groups=seq.shape[1])[:, :, -1]
    out = gdn.causal_conv1d_update(x, state, weight, bias, None)
    torch.testing.assert_close(out, want, rtol=1e-5, atol=1e-6)


def test_conv_token_by_token_equals_one_causal_convolution():
    gen = torch.Generator().manual_seed(4)
    C, K, T = 16, 4, 9
    xs = torch.randn(2, C, T, generator=gen)
    weight = torch.randn(C, K, generator=gen)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(xs, (K - 1, 0)), weight[:, None, :], groups=C)
    for L in (K - 1, K):
        state = torch.zeros(2, C, L)
        got = torch.stack([gdn.causal_conv1d_update(xs[:, :, t].contiguous(), state, weight, None, None)
                           for t in range(T)], dim=2)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
        assert torch.equal(state, xs[:, :, T - L:])


def test_conv_update_matches_third_party_golden():
    z = np.load(GOLDEN_DIR / 'conv1d_update_golden.npz')
    for tag in 'abc':
        state = torch.from_numpy(z[f'{tag}_state0']).clone()
        weight = torch.from_numpy(z[f'{tag}_weight'])
        bias = torch.from_numpy(z[f'{tag}_bias']) if z[f'{tag}_bias'].size else None
        for t in range(3):
            out = gdn.causal_conv1d_update(torch.from_numpy(z[f'{tag}_x{t}']), state, weight, bias, 'silu')
            np.testing.assert_allclose(out.numpy(), z[f'{tag}_out{t}'], rtol=1e-5, atol=1e-6)
            np.testing.assert_array_equal(state.numpy(), z[f'{tag}_state{t + 1}'])


def test_conv_update_rounds_once_for_bf16():
    gen = torch.Generator().manual_seed(5)
    x, state, weight, bias = gdn.conv_make_inputs(2, 8, 8, 4, 4, torch.bfloat16, generator=gen)
    exact = gdn.causal_conv1d_update(x.float(), state.float().clone(), weight.float(), bias.float())
    out = gdn.causal_conv1d_update(x, state, weight, bias)
    assert out.dtype == torch.bfloat16 and state.dtype == torch.bfloat16
    assert torch.equal(out, exact.bfloat16())


# ---- gated RMS normalisation of the read-out -----------------------------------------------------

def test_gated_rmsnorm_closed_form_and_invariants():
    gen = torch.Generator().manual_seed(12)
    o = torch.randn(5, 7, 128, generator=gen) * 3
    z = torch.randn(5, 7, 128, generator=gen)
    w = 1.0 + 0.2 * torch.randn(128, generator=gen)
    y = gdn.gated_rmsnorm(o, z, w, 1e-6)
    od, zd = o.double(), z.double()
    want = w.double() * od / torch.sqrt(od.pow(2).mean(-1, keepdim=True) + 1e-6) * zd / (1 + torch.exp(-zd))
    torch.testing.assert_close(y.double(), want, rtol=1e-5, atol=1e-6)
    # the normalised vector has unit rms; a zero gate gives zero; scale invariance in o (eps aside)
    n = gdn.gated_rmsnorm(o, torch.full_like(z, 50.0), torch.ones(128), 0.0) / 50.0
    torch.testing.assert_close(n.pow(2).mean(-1), torch.ones(5, 7), rtol=1e-5, atol=0)
    assert (gdn.gated_rmsnorm(o, torch.zeros_like(z), w) == 0).all()
    torch.testing.assert_close(gdn.gated_rmsnorm(4 * o, z, w, 0.0), gdn.gated_rmsnorm(o, z, w, 0.0), rtol=1e-5, atol=1e-6)
    assert gdn.gated_rmsnorm(o, z.bfloat16(), w).dtype == torch.bfloat16


def test_gated_rmsnorm_matches_third_party_golden():
    g = np.load(GOLDEN_DIR / 'gated_rmsnorm_golden.npz')
    y = gdn.gated_rmsnorm(torch.from_numpy(g['o']), torch.from_numpy(g['z']), torch.from_numpy(g['weight']), 1e-6)
    np.testing.assert_allclose(y.numpy(), g['y'], rtol=1e-5, atol=1e-6)
