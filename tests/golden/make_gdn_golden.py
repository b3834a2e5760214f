"""Writes tests/golden/gdn_decode_golden.npz from an independent implementation of the gated
delta rule: the eager ``torch_recurrent_gated_delta_rule`` of the locally installed third-party
``transformers`` package (models/qwen3_next/modeling_qwen3_next.py), called with a sequence of
length 1. That function takes [B, T, H, d] tensors, the decay as a log and ungrouped heads, so
the inputs are re-laid out here; it is not part of the reference repository and not needed at
test time (the fixture is committed).

    python tests/golden/make_gdn_golden.py
"""
import sys
from pathlib import Path

import numpy as np
import torch

sys.path.insert(0, str(Path(__file__).resolve().parents[2]))
from oracle.gdn import gdn_make_inputs  # noqa: E402  (input generator only)


def main():
    from transformers.models.qwen3_next.modeling_qwen3_next import torch_recurrent_gated_delta_rule
    fn = getattr(torch_recurrent_gated_delta_rule, '__wrapped__', torch_recurrent_gated_delta_rule)

    gen = torch.Generator().manual_seed(424242)
    B, Hv, Hqk, dk, dv = 2, 4, 2, 128, 128
    q, k, v, g, beta, state = gdn_make_inputs(B, Hv, Hqk, dk, dv, generator=gen)
    rep = Hv // Hqk
    o, new_state = fn(
        q.repeat_interleave(rep, 1)[:, None], k.repeat_interleave(rep, 1)[:, None], v[:, None],
        g.log()[:, None], beta[:, None], initial_state=state.clone(), output_final_state=True)
    out = Path(__file__).with_name('gdn_decode_golden.npz')
    np.savez_compressed(out, q=q.numpy(), k=k.numpy(), v=v.numpy(), g=g.numpy(), beta=beta.numpy(),
                        state=state.numpy(), o=o[:, 0].numpy(), new_state=new_state.numpy())
    print('wrote', out, out.stat().st_size, 'bytes')


if __name__ == '__main__':
    main()
