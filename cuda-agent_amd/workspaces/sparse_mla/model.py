# Task definition: DeepSeek-style sparse-MLA decode attention, eager PyTorch.
#
# Follows the workspace contract of agent_workdir/model.py:9-26 (`Model`, `get_inputs`,
# `get_init_inputs`); this is the fixed side of the pair and the correctness reference that
# utils/verification.py compares the extension against.
#
# Per request b, every head attends to the rows idx[b] of the request's latent KV cache:
#     K_g = kv[b, idx[b]];  s = q[b] @ K_g.T * 192**-0.5;  out = softmax(s) @ K_g[:, :512]
# bf16 inputs, fp32 arithmetic, bf16 output. Index entries < 0 or >= N are padding.
#
# MLA_CONFIG selects the workload: 3 (default) B=64, 128 heads, 32768-row caches (2.4 GB),
# top-k 2048; "small" B=4, 4096-row caches, top-k 512.
import os

import torch
import torch.nn as nn

CONFIGS = {
    '3': dict(batch=64, n_heads=128, n_kv_rows=32768, topk=2048),
    'small': dict(batch=4, n_heads=128, n_kv_rows=4096, topk=512),
}
CONFIG_ID = os.environ.get('MLA_CONFIG', '3')
SEED = 20253
D_QK, D_V = 576, 512
_generator = torch.Generator().manual_seed(SEED)


class Model(nn.Module):

    def __init__(self, n_heads: int, d_qk: int, d_v: int) -> None:
        super().__init__()
        self.n_heads = n_heads
        self.d_qk = d_qk
        self.d_v = d_v
        self.sm_scale = 192 ** -0.5

    def forward(self, q, kv, idx):
        B, N, _ = kv.shape
        out = torch.empty(B, self.n_heads, self.d_v, dtype=torch.bfloat16, device=q.device)
        for b in range(B):                       # one request at a time bounds the temporaries
            valid = (idx[b] >= 0) & (idx[b] < N)
            rows = kv[b, idx[b].clamp(0, N - 1).long()].float()
            s = (q[b].float() @ rows.T) * self.sm_scale
            s = s.masked_fill(~valid[None, :], float('-inf'))
            out[b] = (torch.softmax(s, dim=-1) @ rows[:, :self.d_v]).to(torch.bfloat16)
        return out


def get_inputs():
    # Successive calls continue one seeded stream: every draw is new and the sequence is fixed.
    c = CONFIGS[CONFIG_ID]
    gen = _generator
    B, H, N, topk = c['batch'], c['n_heads'], c['n_kv_rows'], c['topk']
    q = torch.randn(B, H, D_QK, generator=gen).bfloat16()
    kv = torch.empty(B, N, D_QK, dtype=torch.bfloat16)
    for b in range(B):                           # per request, so the fp32 draw stays small
        kv[b] = torch.randn(N, D_QK, generator=gen).bfloat16()
    idx = torch.stack([torch.randperm(N, generator=gen)[:topk] for _ in range(B)]).int()
    return [q, kv, idx]


def get_init_inputs():
    return [CONFIGS[CONFIG_ID]['n_heads'], D_QK, D_V]
