# Task definition: FP8 block-scaled MoE layer, eager PyTorch.
#
# Follows the workspace contract of agent_workdir/model.py:9-26 (`Model`, `get_inputs`,
# `get_init_inputs`); this is the fixed side of the pair and the correctness reference that
# utils/verification.py compares the extension against.
#
# forward(x [T,H] bf16, logits [T,E] fp32) -> out [T,H] bf16 with buffers
#   w13_q [E,2I,H] e4m3 (rows 0..I-1 gate, I..2I-1 up), w13_s [E,2I/128,H/128] fp32,
#   w2_q  [E,H,I]  e4m3,                                  w2_s  [E,H/128,I/128] fp32:
#   route     the 8 largest logits of a token (ties: lower expert id), w = sigmoid normalised
#   quantise  per row and 128 group: scale = max(amax,1e-12) * fp32(1/448), e4m3(clamp(v/scale, +-448))
#   expert    gu = deq(x_q) @ deq(w13[e]).T; h = silu(g)*u; requantise h; y = deq(h_q) @ deq(w2[e]).T
#   combine   out[t] = sum_k w[t,k] * y[t,k], k ascending, fp32 -> bf16
#
# MOE_CONFIG selects the workload: 2 (default) T=64 decode, 4 T=8192 prefill with +2 logit bias
# on 16 experts, "small" a reduced layer (T=64, H=1024, I=512, E=32). Expert weights are generated
# once, from raw random bits (the full layer holds 11.3 GB of them; a normal draw in fp32 and a cast
# would spend minutes on the host): every code takes a random sign, a random 3-bit mantissa and one of
# four consecutive exponents, i.e. magnitudes log-uniform over [0.5, 8) for w13 and [1, 16) for w2
# (rms 3.4 and 6.8, of the order of the 448/sqrt(fan_in) that makes the pre-activations of N(0,1) inputs O(1),
# and outputs of about 0.1, where the harness's atol = rtol = 1e-2 means what it meant for its own example);
# no NaN code can occur. Block scales U(0.5,1.5)/448. The draw runs on the GPU when there is one (the
# harness moves the model there anyway): a second for the full layer against a minute on the host.
import os

import torch
import torch.nn as nn

CONFIGS = {
    '2': dict(tokens=64, hidden=7168, inter=2048, n_experts=256, top_k=8, biased=0),
    '4': dict(tokens=8192, hidden=7168, inter=2048, n_experts=256, top_k=8, biased=16),
    'small': dict(tokens=64, hidden=1024, inter=512, n_experts=32, top_k=8, biased=0),
}
CONFIG_ID = os.environ.get('MOE_CONFIG', '2')
SEED = 20250 + (4 if CONFIG_ID == '4' else 2)
GROUP = 128
_generator = torch.Generator().manual_seed(SEED)
_biased_experts = None


def quantize_groups(v):
    R, C = v.shape
    g = v.float().reshape(R, C // GROUP, GROUP)
    scale = g.abs().amax(dim=-1).clamp_min(1e-12) * (1.0 / 448.0)
    q = (g / scale[:, :, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q.reshape(R, C), scale


def dequantize_groups(q, scale):
    R, C = q.shape
    return (q.float().reshape(R, C // GROUP, GROUP) * scale[:, :, None]).reshape(R, C)


def dequantize_blocks(w_q, w_s):
    s = w_s.repeat_interleave(GROUP, 0).repeat_interleave(GROUP, 1)
    return w_q.float() * s


def random_codes(shape, first_exponent, gen, device='cpu'):
    """e4m3 codes from raw random bits, eight at a time: of every byte drawn, bits 0-2 are the mantissa, bits 3-4
    pick one of the four exponent fields first_exponent .. first_exponent + 3 (values 2^(field - 7) * 1.mmm) and
    bit 5 is the sign."""
    n = 1
    for d in shape:
        n *= d
    assert n % 8 == 0
    codes = torch.empty(n // 8, dtype=torch.int64, device=device)
    step = 1 << 24                                   # 128 MB of codes at a time
    for i in range(0, n // 8, step):
        w = torch.empty(min(step, n // 8 - i), dtype=torch.int64, device=device).random_(generator=gen)
        codes[i:i + step] = ((w & 0x2020202020202020) << 2) | (w & 0x0707070707070707) | \
            ((((w >> 3) & 0x0303030303030303) + first_exponent * 0x0101010101010101) << 3)
    return codes.view(torch.uint8).view(torch.float8_e4m3fn).reshape(shape)


class Model(nn.Module):

    def __init__(self, hidden: int, inter: int, n_experts: int, top_k: int) -> None:
        super().__init__()
        self.hidden, self.inter, self.n_experts, self.top_k = hidden, inter, n_experts, top_k
        device = 'cuda' if torch.cuda.is_available() else 'cpu'
        gen = torch.Generator(device=device).manual_seed(SEED + 1000)
        w13_q = random_codes((n_experts, 2 * inter, hidden), 6, gen, device)
        w2_q = random_codes((n_experts, hidden, inter), 7, gen, device)
        self.register_buffer('w13_q', w13_q)
        self.register_buffer('w13_s', (0.5 + torch.rand(n_experts, 2 * inter // GROUP, hidden // GROUP,
                                                        generator=gen, device=device)) / 448.0)
        self.register_buffer('w2_q', w2_q)
        self.register_buffer('w2_s', (0.5 + torch.rand(n_experts, hidden // GROUP, inter // GROUP,
                                                       generator=gen, device=device)) / 448.0)

    def forward(self, x, logits):
        T, H = x.shape
        I, k = self.inter, self.top_k
        ids = torch.sort(logits, dim=-1, descending=True, stable=True).indices[:, :k]
        score = torch.sigmoid(logits.float()).gather(1, ids)
        weights = score / score.sum(dim=-1, keepdim=True)
        x_dq = dequantize_groups(*quantize_groups(x.float()))
        y = torch.zeros(T, k, H, device=x.device)
        for e in torch.unique(ids).tolist():
            tok, slot = torch.nonzero(ids == e, as_tuple=True)
            gu = x_dq[tok] @ dequantize_blocks(self.w13_q[e], self.w13_s[e]).T
            g, u = gu[:, :I], gu[:, I:]
            h = g / (1.0 + torch.exp(-g)) * u
            y[tok, slot] = dequantize_groups(*quantize_groups(h)) @ dequantize_blocks(self.w2_q[e], self.w2_s[e]).T
        out = torch.zeros(T, H, device=x.device)
        for j in range(k):
            out += weights[:, j:j + 1] * y[:, j]
        return out.to(torch.bfloat16)


def get_inputs():
    # Successive calls continue one seeded stream: every draw is new and the sequence is fixed.
    global _biased_experts
    c = CONFIGS[CONFIG_ID]
    gen = _generator
    x = torch.randn(c['tokens'], c['hidden'], generator=gen).bfloat16()
    logits = torch.randn(c['tokens'], c['n_experts'], generator=gen)
    if c['biased']:
        if _biased_experts is None:              # chosen once per process
            _biased_experts = torch.randperm(c['n_experts'], generator=gen)[:c['biased']]
        logits[:, _biased_experts] += 2.0
    return [x, logits]


def get_init_inputs():
    c = CONFIGS[CONFIG_ID]
    return [c['hidden'], c['inter'], c['n_experts'], c['top_k']]
