"""Oracle for the Gated DeltaNet single-token decode step (test infrastructure only).

Specification restated (workload configs 0 and 1): per request b and value head h, with S the
fp32 ``[dk, dv]`` state, ``g`` the decay itself and q/k shared by ``Hv // Hqk`` consecutive
value heads (head ``h`` reads q/k head ``h // (Hv // Hqk)``)::

    S = g*S;  S += beta * k (v - S^T k)^T;  o = S^T q * dk**-0.5

The reference repository has no implementation of this operator; its model contract
(``Model.forward`` / ``get_inputs`` / ``get_init_inputs``, agent_workdir/model.py:9-26) is
what the functions below are shaped after.

Pinned by (tests/test_oracle_gdn.py):
  * ``gdn_decode_loops_f64``: float64 scalar loops written straight from the recurrence;
  * invariants: beta=0 gives pure decay; g=1, beta=1, |k|=1 gives ``S'^T k == v``;
    the folded single-pass identity ``o = scale*(g*S0^T q + (k.q)*delta)``;
    GQA equals the ungrouped rule fed the repeated q/k heads;
  * a golden fixture written from an independent third-party implementation of the same
    recurrence (tests/golden/make_gdn_golden.py).

``gdn_prestep`` / ``gdn_decode_fused_step`` add the caller's step in front of the recurrence
(L2 normalisation of q and k, decay and write-strength gates). Pinned by: unit norm and scale
invariance of the normalised vectors, ``softplus``/``sigmoid``/``rsqrt`` library routines against
float64 closed forms, limits (a_log -> -inf gives g = 1), and a second golden fixture from the same
third-party function called with its in-kernel L2 normalisation switched on and the gate computed by
library calls (tests/golden/make_gdn_golden.py, ``gdn_fused_golden.npz``).

``gated_rmsnorm`` is the step after the recurrence in the same layer (RMS normalisation of the read-out
over the head dimension, times a weight, times silu of an output gate). Pinned by: the closed form in
float64, unit-rms of the normalised vector, gate z = 0 gives 0, and a golden fixture from the third-party
layer's own norm module in fp32 (``gated_rmsnorm_golden.npz``).

``causal_conv1d_update`` is the step before that one in the same layer (short depthwise causal
convolution over the q|k|v projection, single token, state shifted in place). Pinned by: scalar
loops, the library convolution ``F.conv1d(groups=C)`` over the concatenated sequence, the identity
"feeding a sequence token by token equals one causal convolution of the whole sequence", and a
golden fixture from the third-party layer's own single-token update
(``conv1d_update_golden.npz``, same generator script).
"""

import math

import numpy as np
import torch


def gdn_decode_step(q, k, v, g, beta, state):
    """Vectorised fp32 eager step. Mutates ``state`` in place and returns ``(o, state)``.

    q, k: [B, Hqk, dk]; v: [B, Hv, dv]; g, beta: [B, Hv]; state: [B, Hv, dk, dv] fp32.
    q/k/v may be bf16 or fp32; the arithmetic is fp32.
    """
    B, Hv, dk, dv = state.shape
    rep = Hv // q.shape[1]
    qf = q.float().repeat_interleave(rep, dim=1)
    kf = k.float().repeat_interleave(rep, dim=1)
    vf = v.float()
    state.mul_(g.float()[:, :, None, None])
    u = torch.einsum('bhij,bhi->bhj', state, kf)
    delta = beta.float()[:, :, None] * (vf - u)
    state.add_(kf[:, :, :, None] * delta[:, :, None, :])
    o = torch.einsum('bhij,bhi->bhj', state, qf) * (dk ** -0.5)
    return o, state


L2NORM_EPS = 1e-6


def gdn_prestep(q_raw, k_raw, a, b, a_log, dt_bias):
    """The step in front of the recurrence in Qwen3-Next-style layers (the caller of the path;
    restated from the third-party ``transformers`` layer, models/qwen3_next/modeling_qwen3_next.py:
    ``l2norm`` at :368-371 and the gate lines ``beta = b.sigmoid()``,
    ``g = -A_log.exp() * softplus(a + dt_bias)`` at :659-661, whose recurrent kernel then uses
    ``exp(g)``). Returns ``(q, k, g, beta)`` in the form ``gdn_decode_step`` takes: q, k fp32
    L2-normalised as ``x * rsqrt(sum(x*x) + 1e-6)``, ``g = exp(-exp(a_log) * softplus(a + dt_bias))``
    the decay itself, ``beta = sigmoid(b)``.

    q_raw, k_raw: [B, Hqk, dk] (bf16 or fp32); a, b: [B, Hv]; a_log, dt_bias: [Hv] fp32.
    """
    qf, kf = q_raw.float(), k_raw.float()
    qn = qf * torch.rsqrt((qf * qf).sum(-1, keepdim=True) + L2NORM_EPS)
    kn = kf * torch.rsqrt((kf * kf).sum(-1, keepdim=True) + L2NORM_EPS)
    g = torch.exp(-torch.exp(a_log.float()) * torch.nn.functional.softplus(a.float() + dt_bias.float()))
    beta = torch.sigmoid(b.float())
    return qn, kn, g, beta


def gdn_decode_fused_step(q_raw, k_raw, v, a, b, a_log, dt_bias, state):
    """Pre-step followed by the recurrence; mutates ``state`` and returns ``(o, state)``."""
    qn, kn, g, beta = gdn_prestep(q_raw, k_raw, a, b, a_log, dt_bias)
    return gdn_decode_step(qn, kn, v, g, beta, state)


def gdn_make_raw_inputs(batch, n_v_heads, n_qk_heads, dk=128, dv=128, qkv_dtype=torch.float32,
                        generator=None):
    """Inputs of the fused form: q, k ~ N(0, 1) * U(0.5, 2) per head (not normalised), v ~ N(0,1),
    a, b ~ N(0,1), a_log ~ U(-1, 1), dt_bias ~ U(-1, 1), state ~ N(0, 0.02).
    Returns ``[q_raw, k_raw, v, a, b, a_log, dt_bias, state]``."""
    gen = generator
    q = torch.randn(batch, n_qk_heads, dk, generator=gen) * (0.5 + 1.5 * torch.rand(batch, n_qk_heads, 1, generator=gen))
    k = torch.randn(batch, n_qk_heads, dk, generator=gen) * (0.5 + 1.5 * torch.rand(batch, n_qk_heads, 1, generator=gen))
    v = torch.randn(batch, n_v_heads, dv, generator=gen)
    a = torch.randn(batch, n_v_heads, generator=gen)
    b = torch.randn(batch, n_v_heads, generator=gen)
    a_log = 2 * torch.rand(n_v_heads, generator=gen) - 1
    dt_bias = 2 * torch.rand(n_v_heads, generator=gen) - 1
    state = 0.02 * torch.randn(batch, n_v_heads, dk, dv, generator=gen)
    return [q.to(qkv_dtype), k.to(qkv_dtype), v.to(qkv_dtype), a, b, a_log, dt_bias, state]


def gated_rmsnorm(o, z, weight, eps=1e-6):
    """weight * o * rsqrt(mean(o^2, -1) + eps) * silu(z) in fp32, rounded once to z's dtype.
    o [..., d] fp32 read-out, z [..., d] gate, weight [d]."""
    of = o.float()
    zf = z.float()
    y = weight.float() * (of * torch.rsqrt(of.pow(2).mean(dim=-1, keepdim=True) + eps))
    return (y * (zf * torch.sigmoid(zf))).to(z.dtype)


def gdn_decode_fused_norm_step(q_raw, k_raw, v, a, b, a_log, dt_bias, state, z, norm_w, eps=1e-6):
    """``gdn_decode_fused_step`` followed by ``gated_rmsnorm`` of its read-out. Returns (out, state)."""
    o, state = gdn_decode_fused_step(q_raw, k_raw, v, a, b, a_log, dt_bias, state)
    return gated_rmsnorm(o, z, norm_w, eps), state


def causal_conv1d_update(x, conv_state, weight, bias=None, activation='silu'):
    """x [B,C], conv_state [B,C,L] (oldest first, shifted in place), weight [C,K], bias [C] or None.
    Returns out [B,C] in x's dtype: activation(bias + sum_j weight[:,j] * seq[:, :, L+1-K+j]) with
    seq = [conv_state, x]; fp32 arithmetic, one rounding at the end."""
    L = conv_state.shape[2]
    K = weight.shape[1]
    assert L >= K - 1
    seq = torch.cat([conv_state, x[:, :, None]], dim=2)
    conv_state.copy_(seq[:, :, 1:])
    y = (seq[:, :, L + 1 - K:].float() * weight.float()[None]).sum(dim=2)
    if bias is not None:
        y = y + bias.float()[None]
    if activation == 'silu':
        y = y * torch.sigmoid(y)
    return y.to(x.dtype)


def conv_make_inputs(batch, key_dim, value_dim, state_len=4, kernel_size=4, dtype=torch.bfloat16,
                     generator=None, device='cpu'):
    """x, conv_state ~ N(0,1), weight ~ N(0, 1/K), bias ~ 0.1 N(0,1), all cast to ``dtype``."""
    C = 2 * key_dim + value_dim
    gen = generator
    x = torch.randn(batch, C, generator=gen, device=device).to(dtype)
    conv_state = torch.randn(batch, C, state_len, generator=gen, device=device).to(dtype)
    weight = (torch.randn(C, kernel_size, generator=gen, device=device) * kernel_size ** -0.5).to(dtype)
    bias = (0.1 * torch.randn(C, generator=gen, device=device)).to(dtype)
    return x, conv_state, weight, bias


def gdn_decode_loops_f64(q, k, v, g, beta, state):
    """Scalar float64 loops over numpy arrays; returns ``(o, new_state)``, inputs untouched."""
    q, k, v, g, beta, state = (np.asarray(x, dtype=np.float64) for x in (q, k, v, g, beta, state))
    B, Hv, dk, dv = state.shape
    rep = Hv // q.shape[1]
    S = state.copy()
    o = np.zeros((B, Hv, dv))
    for b in range(B):
        for h in range(Hv):
            hq = h // rep
            for i in range(dk):
                for j in range(dv):
                    S[b, h, i, j] *= g[b, h]
            u = [sum(S[b, h, i, j] * k[b, hq, i] for i in range(dk)) for j in range(dv)]
            for j in range(dv):
                d = beta[b, h] * (v[b, h, j] - u[j])
                for i in range(dk):
                    S[b, h, i, j] += k[b, hq, i] * d
            for j in range(dv):
                o[b, h, j] = sum(S[b, h, i, j] * q[b, hq, i] for i in range(dk)) / math.sqrt(dk)
    return o, S


def gdn_make_inputs(batch, n_v_heads, n_qk_heads, dk=128, dv=128, qkv_dtype=torch.float32,
                    generator=None):
    """Synthetic inputs of the workload: q, k, v ~ N(0,1) with q and k L2-normalised per head in
    fp32 before the cast to ``qkv_dtype``; g = exp(-0.5*softplus(N(0,1))); beta = sigmoid(N(0,1));
    state ~ N(0, 0.02) fp32. Returns ``[q, k, v, g, beta, state]`` on the CPU."""
    gen = generator
    q = torch.randn(batch, n_qk_heads, dk, generator=gen)
    k = torch.randn(batch, n_qk_heads, dk, generator=gen)
    v = torch.randn(batch, n_v_heads, dv, generator=gen)
    q = q / q.norm(dim=-1, keepdim=True)
    k = k / k.norm(dim=-1, keepdim=True)
    g = torch.exp(-0.5 * torch.nn.functional.softplus(torch.randn(batch, n_v_heads, generator=gen)))
    beta = torch.sigmoid(torch.randn(batch, n_v_heads, generator=gen))
    state = 0.02 * torch.randn(batch, n_v_heads, dk, dv, generator=gen)
    return [q.to(qkv_dtype), k.to(qkv_dtype), v.to(qkv_dtype), g, beta, state]


def gdn_close(actual, expected, rtol=1e-3):
    """The fp32 tolerance of this operator: |a-b| <= rtol*|b| + rtol*rms(b).

    A pure relative bound is ill-posed because outputs cross zero; the absolute floor is the
    same fraction of the tensor's RMS."""
    a = actual.double()
    e = expected.double()
    atol = rtol * e.pow(2).mean().sqrt()
    return bool(((a - e).abs() <= rtol * e.abs() + atol).all())
