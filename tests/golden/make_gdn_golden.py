"""Writes tests/golden/gdn_decode_golden.npz (and the two fixtures described further down, for the
fused pre-step and for the convolution update) from an independent implementation of the gated
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

    # fused form: raw q/k normalised inside the third-party function (use_qk_l2norm_in_kernel),
    # log-decay from library calls as in that layer's forward
    from oracle.gdn import gdn_make_raw_inputs
    gen = torch.Generator().manual_seed(434343)
    qr, kr, v, a, b, a_log, dt_bias, state = gdn_make_raw_inputs(B, Hv, Hqk, dk, dv, generator=gen)
    log_g = -a_log.float().exp() * torch.nn.functional.softplus(a.float() + dt_bias)
    o, new_state = fn(
        qr.repeat_interleave(rep, 1)[:, None], kr.repeat_interleave(rep, 1)[:, None], v[:, None],
        log_g[:, None], b.sigmoid()[:, None], initial_state=state.clone(), output_final_state=True,
        use_qk_l2norm_in_kernel=True)
    out = Path(__file__).with_name('gdn_fused_golden.npz')
    np.savez_compressed(out, q=qr.numpy(), k=kr.numpy(), v=v.numpy(), a=a.numpy(), b=b.numpy(),
                        a_log=a_log.numpy(), dt_bias=dt_bias.numpy(), state=state.numpy(),
                        o=o[:, 0].numpy(), new_state=new_state.numpy())
    print('wrote', out, out.stat().st_size, 'bytes')

    # the layer's single-token convolution update (fp32; state of K and of K-1 columns, with and
    # without bias): three consecutive tokens through the third-party function
    from transformers.models.qwen3_next.modeling_qwen3_next import causal_conv1d_update
    from oracle.gdn import conv_make_inputs
    gen = torch.Generator().manual_seed(454545)
    arrays = {}
    for tag, L, K, with_bias in (('a', 4, 4, True), ('b', 3, 4, False), ('c', 2, 2, True)):
        x, conv_state, weight, bias = conv_make_inputs(2, 8, 16, L, K, torch.float32, generator=gen)
        xs = [x, torch.randn(x.shape, generator=gen), torch.randn(x.shape, generator=gen)]
        arrays.update({f'{tag}_state0': conv_state.numpy().copy(), f'{tag}_weight': weight.numpy(),
                       f'{tag}_bias': bias.numpy() if with_bias else np.zeros(0, np.float32)})
        for t, xt in enumerate(xs):
            y = causal_conv1d_update(xt[:, :, None], conv_state, weight, bias if with_bias else None, 'silu')
            arrays.update({f'{tag}_x{t}': xt.numpy(), f'{tag}_out{t}': y[:, :, 0].numpy(),
                           f'{tag}_state{t + 1}': conv_state.numpy().copy()})
    out = Path(__file__).with_name('conv1d_update_golden.npz')
    np.savez_compressed(out, **arrays)
    print('wrote', out, out.stat().st_size, 'bytes')

    # the layer's gated RMS norm (fp32 module: no intermediate roundings)
    from transformers.models.qwen3_next.modeling_qwen3_next import Qwen3NextRMSNormGated
    gen = torch.Generator().manual_seed(474747)
    norm = Qwen3NextRMSNormGated(128, eps=1e-6)
    with torch.no_grad():
        norm.weight.copy_(1.0 + 0.1 * torch.randn(128, generator=gen))
        o = torch.randn(6, 128, generator=gen) * torch.exp(torch.randn(6, 1, generator=gen))
        z = torch.randn(6, 128, generator=gen) * 2
        y = norm(o, z)
    out = Path(__file__).with_name('gated_rmsnorm_golden.npz')
    np.savez_compressed(out, o=o.numpy(), z=z.numpy(), weight=norm.weight.detach().numpy(), y=y.numpy())
    print('wrote', out, out.stat().st_size, 'bytes')


if __name__ == '__main__':
    main()
