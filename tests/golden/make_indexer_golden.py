"""Writes tests/golden/indexer_golden.npz from the indexer of the locally installed third-party ``transformers``
package (models/deepseek_v32/modeling_deepseek_v32.py, ``DeepseekV32Indexer``), one decode step per request:
the module's own projections and rotary embedding produce the query heads, the key row and the per-head weights;
the fixture stores those (what a scoring kernel receives) together with the top-k positions the module returns.
The module is not part of the reference repository and is not needed at test time.

    python tests/golden/make_indexer_golden.py
"""
from pathlib import Path
from types import SimpleNamespace

import numpy as np
import torch


def main():
    from transformers.models.deepseek_v32 import modeling_deepseek_v32 as m
    gen = torch.Generator().manual_seed(484848)
    B, T, hidden, Hi, D, rope, topk, qlora = 3, 96, 64, 32, 128, 64, 24, 48
    cfg = SimpleNamespace(hidden_size=hidden, index_n_heads=Hi, index_head_dim=D, qk_rope_head_dim=rope,
                          index_topk=topk, q_lora_rank=qlora)
    idx = m.DeepseekV32Indexer(cfg, layer_idx=0)
    with torch.no_grad():
        for p in idx.parameters():
            p.copy_(torch.randn(p.shape, generator=gen) * (0.3 if p.dim() > 1 else 1.0))
        # a "sequence" of T positions per request processed at once; the last position's row is the decode step
        hs = torch.randn(B, T, hidden, generator=gen)
        q_resid = torch.randn(B, T, qlora, generator=gen)
        ang = torch.rand(B, T, rope // 2, generator=gen) * 6.28
        cos, sin = torch.cat([ang.cos(), ang.cos()], -1), torch.cat([ang.sin(), ang.sin()], -1)
        position_ids = torch.arange(T)[None].expand(B, T)
        got = idx(hs, q_resid, (cos, sin), None, position_ids, None)           # [B, T, topk]
        # the tensors a scoring kernel receives for the last position, from the module's own submodules
        q = idx.wq_b(q_resid).view(B, T, Hi, D)
        q_rot, q_pass = torch.split(q, [rope, D - rope], dim=-1)
        k = idx.k_norm(idx.wk(hs)).unsqueeze(2)
        k_rot, k_pass = torch.split(k, [rope, D - rope], dim=-1)
        q_rot, k_rot = m.apply_rotary_pos_emb(q_rot, k_rot, cos, sin, unsqueeze_dim=2)
        q = torch.cat([q_rot, q_pass], dim=-1)
        k = torch.cat([k_rot, k_pass], dim=-1).squeeze(2)
        w = idx.weights_proj(hs).float() * Hi ** -0.5
    out = Path(__file__).with_name('indexer_golden.npz')
    np.savez_compressed(out, q=q[:, -1].numpy(), k=k.numpy(), w=w[:, -1].numpy(),
                        topk=np.sort(got[:, -1].numpy(), axis=-1), scale=np.array([idx.softmax_scale], np.float32))
    print('wrote', out, out.stat().st_size, 'bytes')


if __name__ == '__main__':
    main()
