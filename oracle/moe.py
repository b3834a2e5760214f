"""Oracle for the FP8 block-scaled MoE layer (test infrastructure only).

Specification restated (workload configs 2 and 4): ``forward(x[T,H] bf16, logits[T,E] fp32) ->
out[T,H] bf16`` with expert buffers ``w13_q[E,2I,H]`` e4m3 (rows 0..I-1 gate, I..2I-1 up),
``w13_s[E,2I/128,H/128]`` fp32, ``w2_q[E,H,I]`` e4m3, ``w2_s[E,H/128,I/128]`` fp32:

  route      s = sigmoid(logits); the 8 experts of a token are its 8 largest logits (ties: the
             lower expert id), listed in that order; w = s[ids] / sum(s[ids])
  sort       stable counting sort of the T*8 (token, slot) pairs by expert id
  quantise   per row and 128-wide group: scale = max(amax, 1e-12) * fp32(1/448),
             q = e4m3_rne(clamp(v / scale, -448, 448))
             (a multiply by the rounded reciprocal, not a division by 448: eager PyTorch
             evaluates `tensor / 448.0` that way on the GPU but not on the CPU, and with bf16
             inputs v/scale often sits exactly on a rounding tie, where one ulp of the scale
             decides the code)
  expert     gu = deq(x_q) @ deq(w13[e]).T ; h = silu(g) * u ; h_q, h_s = quantise(h) ;
             y = deq(h_q) @ deq(w2[e]).T                    (fp32)
  combine    out[t] = sum_k w[t,k] * y[t,k], k ascending, fp32 -> bf16

Ranking by logit equals ranking by an exact sigmoid and does not depend on how a particular
sigmoid implementation rounds. The reference repository has no implementation of this operator;
only its model contract (agent_workdir/model.py:9-26) shapes the functions below.

``route_grouped`` is the router a DeepSeek-V3-style layer uses in place of ``route`` (group-limited
choice with a selection bias; no counterpart in the reference repository). Pinned by scalar loops
on small sizes, by the reduction to ``route`` when there is one group and no bias, by its
invariants (chosen experts lie in exactly topk_group groups, weights sum to the scaling factor),
and by a golden fixture written from the third-party ``transformers`` router
(tests/golden/make_router_golden.py). ``rmsnorm_bf16`` is the norm in front of the layer (its output is what the layer quantises and what the router
projects); pinned by a float64 closed form within bf16 rounding and by a fixture from the third-party
``DeepseekV3RMSNorm`` module in bf16 (``rmsnorm_golden.npz``, same generator script as the router's).
``router_logits`` is the projection in front of it, pinned by a float64
product and by the same fixture's logits.

``moe_forward_shared`` adds the shared expert of such a layer; it is built from ``moe_forward`` itself
and pinned by a float64 dense evaluation of the same sum on a tiny shape.

The UE8M0 form of the layer (``pow2_scales``; no counterpart in the reference repository) changes one
line of the specification: an activation scale is the smallest power of two >= amax/448 instead of
amax * fp32(1/448); weight scales are given as powers of two. Pinned by: ``pow2_ceil`` against float64
``2**ceil(log2 v)`` and on exact powers of two and their neighbours; scale in [amax/448, 2*amax/448);
the group maximum maps to a code in [224, 448]; division by the scale exact (codes equal the e4m3
rounding of an exactly scaled value); the dense float64 layer evaluation with those scales.

Pinned by (tests/test_oracle_moe.py):
  * e4m3: the 256-entry decode table against torch's float8_e4m3fn and the closed form; the
    encoder against torch's cast on every representable value, every midpoint and random
    floats; idempotence; the group maximum maps to +-448;
  * routing/sort: torch.topk / stable argsort / bincount, brute force on tiny sizes, and the
    permutation invariants;
  * GEMMs/combine: float64 dense matmul on dequantised tiny shapes; the exact-integer case;
    the single-expert (k=1, w=1) case as a plain MLP; block-scale linearity.
"""

import numpy as np
import torch

E4M3_MAX = 448.0
GROUP = 128
AMAX_FLOOR = 1e-12


# ---------------------------------------------------------------------------------- e4m3 codec

def e4m3_decode_table():
    """float32[256]: value of every OCP e4m3fn code (0x7f / 0xff are NaN), from the closed form."""
    out = np.zeros(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp = (code >> 3) & 0xF
        man = code & 0x7
        if exp == 0xF and man == 0x7:
            val = np.nan
        elif exp == 0:
            val = man * 2.0 ** -9
        else:
            val = (1.0 + man / 8.0) * 2.0 ** (exp - 7)
        out[code] = sign * val
    return out


def e4m3_encode(x):
    """Round-to-nearest-even encode of a float32 array to e4m3fn codes (uint8), saturating at
    +-448 (numpy, independent of torch's cast)."""
    x = np.asarray(x, dtype=np.float32)
    a = np.minimum(np.abs(x), np.float32(E4M3_MAX)).astype(np.float64)
    # exponent of the target binade; subnormals share the step 2^-9
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -20)))
    e = np.maximum(e, -6.0)
    step = 2.0 ** (e - 3)
    qv = np.rint(a / step) * step            # np.rint rounds half to even
    qv = np.minimum(qv, E4M3_MAX)
    # value -> code
    e2 = np.floor(np.log2(np.maximum(qv, 2.0 ** -20)))
    normal = qv >= 2.0 ** -6
    exp_field = np.where(normal, e2 + 7, 0).astype(np.int64)
    man_field = np.where(normal, np.rint((qv / 2.0 ** np.where(normal, e2, 0) - 1.0) * 8),
                         np.rint(qv * 2.0 ** 9)).astype(np.int64)
    code = (exp_field << 3) | man_field
    code = np.where(np.signbit(x), code | 0x80, code)
    return code.astype(np.uint8)


def pow2_ceil(v):
    """The smallest power of two >= v, for positive fp32 v, exactly (frexp: v = m * 2^e, 0.5 <= m < 1)."""
    m, e = torch.frexp(v.float())
    return torch.ldexp(torch.ones_like(m), torch.where(m == 0.5, e - 1, e))


def quantize_groups(v, pow2=False):
    """Per-row, per-128-group e4m3 quantisation of a 2-D fp32 tensor.
    Returns (codes float8_e4m3fn [R,C], scales fp32 [R,C/128]). ``pow2``: the UE8M0 convention, scale =
    the smallest power of two >= amax/448."""
    R, C = v.shape
    g = v.float().reshape(R, C // GROUP, GROUP)
    amax = g.abs().amax(dim=-1).clamp_min(AMAX_FLOOR)
    if pow2:
        # amax/448 in float64 is not exact, but a power of two p satisfies p >= amax/448 iff 448*p >= amax,
        # and 448*p is exact: take the candidate from the rounded quotient and correct it by one step
        p = pow2_ceil((amax.double() / E4M3_MAX).float())
        p = torch.where(p.double() * E4M3_MAX < amax.double(), p * 2, p)
        p = torch.where((p.double() / 2) * E4M3_MAX >= amax.double(), p / 2, p)
        scale = p
    else:
        scale = amax * (1.0 / E4M3_MAX)
    q = (g / scale[:, :, None]).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return q.reshape(R, C), scale


def dequantize_groups(q, scale):
    R, C = q.shape
    return (q.float().reshape(R, C // GROUP, GROUP) * scale[:, :, None]).reshape(R, C)


def dequantize_blocks(w_q, w_s):
    """w_q [N,K] e4m3 with one fp32 scale per 128x128 block, w_s [N/128, K/128] -> fp32 [N,K]."""
    N, K = w_q.shape
    s = w_s.repeat_interleave(GROUP, 0).repeat_interleave(GROUP, 1)
    return w_q.float() * s[:N, :K]


# ------------------------------------------------------------------------------ routing / sort

def route(logits, top_k=8):
    """ids int32 [T,k] (descending logit, ties to the lower id), weights fp32 [T,k]."""
    order = torch.sort(logits, dim=-1, descending=True, stable=True).indices[:, :top_k]
    score = torch.sigmoid(logits.float()).gather(1, order)
    return order.int(), score / score.sum(dim=-1, keepdim=True)


def rmsnorm_bf16(x, weight, eps=1e-6):
    """The RMS norm of a bf16 layer as the third-party layers evaluate it: fp32 statistics, the normalised value
    rounded to bf16, times the bf16 weight, rounded to bf16. x [R,C] bf16, weight [C] bf16 -> [R,C] bf16."""
    xf = x.float()
    n = (xf * (1.0 / torch.sqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps))).to(x.dtype)
    return weight * n


def router_logits(x, w):
    """logits [T,E] fp32 = x [T,H] (bf16 or fp32, taken to fp32) @ w [E,H]^T (fp32), as the third-party
    router computes them (``F.linear`` of the two fp32 casts)."""
    return x.float() @ w.float().T


def split_bf16x3(w):
    """w fp32 -> planes [3, ...] bf16 with planes.float().sum(0) == w exactly: hi = w with the lower 16 bits cleared,
    mid = (w - hi) with the lower 16 bits cleared, lo = w - hi - mid (8 significant bits are left: a bf16 number)."""
    bits = w.contiguous().view(torch.int32)
    hi = (bits & -65536).view(torch.float32)
    r1 = w - hi
    mid = (r1.contiguous().view(torch.int32) & -65536).view(torch.float32)
    lo = r1 - mid
    return torch.stack([hi, mid, lo]).bfloat16()


def route_grouped(logits, bias, top_k, n_group, topk_group, normalise=True, routed_scaling_factor=1.0):
    """Group-limited routing with a selection bias.

    score = sigmoid(logits); choice = score + bias. A group is a run of E/n_group consecutive experts and
    is valued by the sum of its 2 largest choice values; the topk_group best groups stay (ties to the lower
    group). ids int32 [T,k]: the top_k largest choice values among the experts that stay, descending, ties
    to the lower id. weights fp32 [T,k] = score[ids] (/ (sum + 1e-20) if ``normalise``) * scaling factor.
    Returns (ids, weights, choice) - ``choice`` fp32 [T,E] lets a checker see how close a decision was."""
    T, E = logits.shape
    score = torch.sigmoid(logits.float())
    choice = score if bias is None else score + bias.float()[None]
    grouped = choice.view(T, n_group, E // n_group)
    value = grouped.topk(min(2, E // n_group), dim=-1).values.sum(dim=-1)
    stay_groups = torch.sort(value, dim=-1, descending=True, stable=True).indices[:, :topk_group]
    stay = torch.zeros(T, n_group, dtype=torch.bool).scatter_(1, stay_groups, True)
    masked = grouped.masked_fill(~stay[:, :, None], float('-inf')).reshape(T, E)
    ids = torch.sort(masked, dim=-1, descending=True, stable=True).indices[:, :top_k]
    w = score.gather(1, ids)
    if normalise:
        w = w / (w.sum(dim=-1, keepdim=True) + 1e-20)
    return ids.int(), w * routed_scaling_factor, choice


def sort_pairs(ids, n_experts):
    """Stable counting sort of the flattened (token, slot) pairs by expert.
    Returns sorted_pairs int32 [T*k] (flat pair index at each sorted position),
    pair_pos int32 [T*k] (its inverse) and expert_offsets int32 [E+1]."""
    flat = ids.reshape(-1).long()
    sorted_pairs = torch.sort(flat, stable=True).indices
    counts = torch.bincount(flat, minlength=n_experts)
    offsets = torch.zeros(n_experts + 1, dtype=torch.long)
    offsets[1:] = counts.cumsum(0)
    pair_pos = torch.empty_like(sorted_pairs)
    pair_pos[sorted_pairs] = torch.arange(flat.numel())
    return sorted_pairs.int(), pair_pos.int(), offsets.int()


# ----------------------------------------------------------------------------------- the layer

def silu(x):
    return x / (1.0 + torch.exp(-x))


def moe_forward(x, logits, w13_q, w13_s, w2_q, w2_s, top_k=8, out_dtype=torch.bfloat16,
                return_intermediates=False, pow2_scales=False):
    """``pow2_scales``: the UE8M0 form of the layer, activations quantised with power-of-two scales (the
    weight scales handed in must be powers of two as well; checked)."""
    if pow2_scales:
        for ws in (w13_s, w2_s):
            assert torch.equal(ws, pow2_ceil(ws)), 'UE8M0 form: weight scales must be powers of two'
    T, H = x.shape
    E, I2, _ = w13_q.shape
    I = I2 // 2
    ids, weights = route(logits, top_k)
    x_q, x_s = quantize_groups(x.float(), pow2_scales)
    x_dq = dequantize_groups(x_q, x_s)
    y = torch.zeros(T, top_k, H)
    h_q_all = torch.zeros(T, top_k, I, dtype=torch.float8_e4m3fn)
    h_s_all = torch.zeros(T, top_k, I // GROUP)
    for e in torch.unique(ids).tolist():
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        w13 = dequantize_blocks(w13_q[e], w13_s[e])
        gu = x_dq[tok] @ w13.T
        h = silu(gu[:, :I]) * gu[:, I:]
        h_q, h_s = quantize_groups(h, pow2_scales)
        h_q_all[tok, slot] = h_q
        h_s_all[tok, slot] = h_s
        y[tok, slot] = dequantize_groups(h_q, h_s) @ dequantize_blocks(w2_q[e], w2_s[e]).T
    out = torch.zeros(T, H)
    for k in range(top_k):
        out += weights[:, k:k + 1] * y[:, k]
    out = out.to(out_dtype)
    if return_intermediates:
        return out, dict(ids=ids, weights=weights, x_q=x_q, x_s=x_s, h_q=h_q_all, h_s=h_s_all, y=y)
    return out


def moe_forward_shared(x, logits, w13_q, w13_s, w2_q, w2_s, sw13_q, sw13_s, sw2_q, sw2_s, top_k=8,
                       out_dtype=torch.bfloat16, pow2_scales=False):
    """The layer plus a shared expert: one more block-scaled MLP (sw13_q [2*Is,H], sw13_s, sw2_q [H,Is],
    sw2_s) applied to every token with weight 1, added in fp32 after the routed experts' weighted sum.
    The shared expert is evaluated by the same stage functions: a layer of one expert chosen by every
    token with routing weight s/s = 1."""
    routed = moe_forward(x, logits, w13_q, w13_s, w2_q, w2_s, top_k, torch.float32, pow2_scales=pow2_scales)
    shared = moe_forward(x, torch.zeros(x.shape[0], 1), sw13_q[None], sw13_s[None], sw2_q[None], sw2_s[None],
                         1, torch.float32, pow2_scales=pow2_scales)
    return (routed + shared).to(out_dtype)


# ---------------------------------------------------------------------------- synthetic inputs

def random_e4m3(shape, generator=None, device='cpu'):
    """Uniformly random e4m3 codes with the two NaN codes excluded: magnitudes are log-uniform
    over the format's range, so a 128-term dot product is dominated by its few largest terms."""
    codes = torch.randint(0, 256, shape, dtype=torch.uint8, generator=generator, device=device)
    codes = torch.where((codes & 0x7F) == 0x7F, codes ^ 1, codes)
    return codes.view(torch.float8_e4m3fn)


def normal_e4m3(shape, std, generator=None, device='cpu'):
    """e4m3 codes of N(0, std) samples, clamped to +-448."""
    v = torch.randn(shape, generator=generator, device=device) * std
    return v.clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)


def moe_make_weights(n_experts, hidden, inter, generator=None, device='cpu', pow2_scales=False):
    """Expert weights: e4m3 codes of N(0, 448/sqrt(fan_in)) and 128x128 block scales
    ~ U(0.5, 1.5)/448, so that a dequantised weight is about N(0, 1/fan_in) and the
    pre-activations of N(0,1) inputs are O(1). (The workload leaves the code distribution open.)
    ``pow2_scales``: every scale rounded up to a power of two (2^-9 or 2^-8)."""
    gen = generator
    w13_q = normal_e4m3((n_experts, 2 * inter, hidden), E4M3_MAX / hidden ** 0.5, gen, device)
    w2_q = normal_e4m3((n_experts, hidden, inter), E4M3_MAX / inter ** 0.5, gen, device)
    w13_s = (0.5 + torch.rand(n_experts, 2 * inter // GROUP, hidden // GROUP, generator=gen,
                              device=device)) / 448.0
    w2_s = (0.5 + torch.rand(n_experts, hidden // GROUP, inter // GROUP, generator=gen,
                             device=device)) / 448.0
    if pow2_scales:
        w13_s, w2_s = pow2_ceil(w13_s), pow2_ceil(w2_s)
    return w13_q, w13_s, w2_q, w2_s


def moe_make_inputs(tokens, hidden, n_experts, generator=None, device='cpu', biased_experts=None,
                    bias=2.0):
    x = torch.randn(tokens, hidden, generator=generator, device=device).bfloat16()
    logits = torch.randn(tokens, n_experts, generator=generator, device=device)
    if biased_experts is not None:
        logits[:, biased_experts] += bias
    return [x, logits]


def rel_rms_error(actual, expected):
    a = actual.double()
    e = expected.double()
    return ((a - e).abs().max() / e.pow(2).mean().sqrt()).item()
