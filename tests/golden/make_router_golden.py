"""Writes tests/golden/router_golden.npz from the router of the locally installed third-party
``transformers`` package (models/deepseek_v3/modeling_deepseek_v3.py, ``DeepseekV3TopkRouter``):
hidden states, router weight and selection bias in, fp32 logits, chosen experts and their weights out.
That class is not part of the reference repository and is not needed at test time (the fixture is
committed). torch.topk(sorted=False) leaves the order of the chosen experts open, so the fixture
stores them sorted by expert id.

    python tests/golden/make_router_golden.py
"""
from pathlib import Path
from types import SimpleNamespace

import numpy as np
import torch


def main():
    from transformers.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3TopkRouter
    arrays = {}
    gen = torch.Generator().manual_seed(464646)
    for tag, (T, H, E, k, G, kg, norm, scale) in {'a': (48, 64, 256, 8, 8, 4, True, 2.5),
                                                  'b': (33, 32, 64, 6, 4, 2, False, 1.0),
                                                  'c': (16, 32, 32, 4, 1, 1, True, 1.0)}.items():
        cfg = SimpleNamespace(num_experts_per_tok=k, num_local_experts=E, hidden_size=H, routed_scaling_factor=scale,
                              n_group=G, topk_group=kg, norm_topk_prob=norm)
        router = DeepseekV3TopkRouter(cfg)
        with torch.no_grad():
            router.weight.copy_(torch.randn(E, H, generator=gen) * H ** -0.5)
            router.e_score_correction_bias.copy_(0.1 * torch.randn(E, generator=gen))
            hidden = torch.randn(T, H, generator=gen).bfloat16()
            logits, weights, ids = router(hidden)
        order = ids.argsort(dim=-1)
        arrays.update({f'{tag}_hidden': hidden.float().numpy(), f'{tag}_weight': router.weight.detach().numpy(),
                       f'{tag}_bias': router.e_score_correction_bias.numpy(), f'{tag}_logits': logits.numpy(),
                       f'{tag}_ids': ids.gather(1, order).int().numpy(),
                       f'{tag}_weights': weights.gather(1, order).numpy(),
                       f'{tag}_params': np.array([k, G, kg, int(norm)], np.int32),
                       f'{tag}_scale': np.array([scale], np.float32)})
    out = Path(__file__).with_name('router_golden.npz')
    np.savez_compressed(out, **arrays)
    print('wrote', out, out.stat().st_size, 'bytes')

    # the bf16 RMS norm in front of the layer
    from transformers.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3RMSNorm
    gen = torch.Generator().manual_seed(494949)
    norm = DeepseekV3RMSNorm(256, eps=1e-6).bfloat16()
    with torch.no_grad():
        norm.weight.copy_((1.0 + 0.2 * torch.randn(256, generator=gen)).bfloat16())
        x = (torch.randn(12, 256, generator=gen) * torch.exp(torch.randn(12, 1, generator=gen))).bfloat16()
        y = norm(x)
    out = Path(__file__).with_name('rmsnorm_golden.npz')
    np.savez_compressed(out, x=x.float().numpy(), weight=norm.weight.detach().float().numpy(), y=y.float().numpy())
    print('wrote', out, out.stat().st_size, 'bytes')


if __name__ == '__main__':
    main()
