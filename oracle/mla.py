"""Oracle for sparse-MLA decode attention (test infrastructure only).

Specification restated (workload config 3): per request b, all heads attend to the rows of the
request's latent cache selected by ``idx[b]``::

    K_g = kv[b, idx[b]]                      [topk, 576]
    s   = q[b] @ K_g.T * sm_scale            [heads, topk]     sm_scale = 192**-0.5
    out = softmax(s) @ K_g[:, :512]          [heads, 512] -> bf16

bf16 inputs are upcast and all arithmetic is fp32. Index values < 0 or >= N are padding and
take no part in the softmax. The reference repository has no implementation of this operator;
only its model contract (agent_workdir/model.py:9-26) shapes the functions below.

Pinned by (tests/test_oracle_mla.py):
  * ``sparse_mla_loops_f64``: float64 scalar loops written straight from the definition;
  * library special case: idx = arange(N) equals ``scaled_dot_product_attention`` with one
    shared KV head;
  * invariants: permutation of idx, all-equal V rows, shift invariance, split-and-merge by
    log-sum-exp.
"""

import math

import numpy as np
import torch

D_QK = 576
D_V = 512
SM_SCALE = 192 ** -0.5


def sparse_mla_decode(q, kv, idx, sm_scale=SM_SCALE, out_dtype=torch.bfloat16):
    """q [B,H,576], kv [B,N,576], idx [B,topk] int32 -> out [B,H,512] (fp32 math)."""
    B, H, _ = q.shape
    N = kv.shape[1]
    valid = (idx >= 0) & (idx < N)
    safe = idx.clamp(0, N - 1).long()
    kg = torch.gather(kv, 1, safe[:, :, None].expand(-1, -1, kv.shape[2])).float()
    s = torch.einsum('bhd,bkd->bhk', q.float(), kg) * sm_scale
    s = s.masked_fill(~valid[:, None, :], float('-inf'))
    p = torch.softmax(s, dim=-1)
    out = torch.einsum('bhk,bkd->bhd', p, kg[:, :, :D_V])
    return out.to(out_dtype)


def sparse_mla_loops_f64(q, kv, idx, sm_scale=SM_SCALE):
    q = np.asarray(q, dtype=np.float64)
    kv = np.asarray(kv, dtype=np.float64)
    B, H, D = q.shape
    N = kv.shape[1]
    dv = min(D_V, D)
    out = np.zeros((B, H, dv))
    for b in range(B):
        rows = [int(i) for i in idx[b] if 0 <= int(i) < N]
        for h in range(H):
            scores = [sum(q[b, h, d] * kv[b, r, d] for d in range(D)) * sm_scale for r in rows]
            mx = max(scores)
            w = [math.exp(s - mx) for s in scores]
            tot = sum(w)
            for j in range(dv):
                out[b, h, j] = sum(wi * kv[b, r, j] for wi, r in zip(w, rows)) / tot
    return out


def mla_make_inputs(batch, n_heads, n_kv_rows, topk, generator=None, device='cpu'):
    """q, kv ~ N(0,1) cast to bf16; idx = the first topk entries of a per-request random
    permutation of the cache rows (unsorted, no repeats), int32."""
    gen = generator
    q = torch.randn(batch, n_heads, D_QK, generator=gen, device=device).bfloat16()
    kv = torch.randn(batch, n_kv_rows, D_QK, generator=gen, device=device).bfloat16()
    idx = torch.stack([torch.randperm(n_kv_rows, generator=gen, device=device)[:topk]
                       for _ in range(batch)]).int()
    return [q, kv, idx]


def rel_rms_error(actual, expected):
    """max |a - e| / rms(e): the figure the 2e-2 bound of this operator is stated on."""
    a = actual.double()
    e = expected.double()
    return ((a - e).abs().max() / e.pow(2).mean().sqrt()).item()
