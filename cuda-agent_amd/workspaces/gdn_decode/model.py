# Task definition: Gated DeltaNet single-token decode step, eager PyTorch.
#
# Follows the workspace contract of agent_workdir/model.py:9-26 (`Model`, `get_inputs`,
# `get_init_inputs`); this is the fixed side of the pair and the correctness reference that
# utils/verification.py compares the extension against.
#
# Per request b and value head h (q/k head h // (Hv // Hqk)), with S the fp32 [dk, dv] state:
#     S = g*S;  S += beta * k (v - S^T k)^T;  o = S^T q * dk**-0.5
# `g` is the decay factor itself. The state tensor is updated in place and returned with o.
#
# GDN_CONFIG selects the workload: 0 (default) B=1, 16 heads, fp32 q/k/v;
# 1 B=256, 32 value heads over 16 q/k heads, bf16 q/k/v, 537 MB of state.
import os

import torch
import torch.nn as nn

CONFIGS = {
    0: dict(batch=1, n_v_heads=16, n_qk_heads=16, dk=128, dv=128, qkv_dtype=torch.float32),
    1: dict(batch=256, n_v_heads=32, n_qk_heads=16, dk=128, dv=128, qkv_dtype=torch.bfloat16),
}
CONFIG_ID = int(os.environ.get('GDN_CONFIG', '0'))
SEED = 20250 + CONFIG_ID
_generator = torch.Generator().manual_seed(SEED)


class Model(nn.Module):

    def __init__(self, n_v_heads: int, n_qk_heads: int, dk: int, dv: int) -> None:
        super().__init__()
        self.n_v_heads = n_v_heads
        self.n_qk_heads = n_qk_heads
        self.dk = dk
        self.dv = dv

    def forward(self, q, k, v, g, beta, state):
        rep = self.n_v_heads // self.n_qk_heads
        q = q.float().repeat_interleave(rep, dim=1)
        k = k.float().repeat_interleave(rep, dim=1)
        v = v.float()
        state.mul_(g[:, :, None, None])
        u = (state * k[:, :, :, None]).sum(dim=2)
        delta = beta[:, :, None] * (v - u)
        state.add_(k[:, :, :, None] * delta[:, :, None, :])
        o = (state * q[:, :, :, None]).sum(dim=2) * self.dk ** -0.5
        return o, state


def get_inputs():
    # Successive calls continue one seeded stream: every draw is new and the sequence is fixed.
    c = CONFIGS[CONFIG_ID]
    gen = _generator
    B, Hv, Hqk, dk, dv = c['batch'], c['n_v_heads'], c['n_qk_heads'], c['dk'], c['dv']
    q = torch.randn(B, Hqk, dk, generator=gen)
    k = torch.randn(B, Hqk, dk, generator=gen)
    v = torch.randn(B, Hv, dv, generator=gen)
    q = q / q.norm(dim=-1, keepdim=True)
    k = k / k.norm(dim=-1, keepdim=True)
    g = torch.exp(-0.5 * torch.log1p(torch.exp(torch.randn(B, Hv, generator=gen))))
    beta = torch.sigmoid(torch.randn(B, Hv, generator=gen))
    state = 0.02 * torch.randn(B, Hv, dk, dv, generator=gen)
    dt = c['qkv_dtype']
    return [q.to(dt), k.to(dt), v.to(dt), g, beta, state]


def get_init_inputs():
    c = CONFIGS[CONFIG_ID]
    return [c['n_v_heads'], c['n_qk_heads'], c['dk'], c['dv']]
