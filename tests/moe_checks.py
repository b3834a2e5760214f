"""Checks shared by the GPU parity tests of the FP8 MoE layer: distances between e4m3 codes, the oracle's down
projection on given codes, and the settlement of requantised codes on which two fp32 evaluations disagree."""
import torch

from oracle import moe


def code_steps(a, b):
    """Distance between e4m3 codes in steps of the format: codes are sign-magnitude, so the magnitude bits count
    the steps from zero, +0 and -0 coincide and the smallest values of either sign are two steps apart."""
    def signed(c):
        c = c.view(torch.uint8).int()
        return torch.where(c >= 128, -(c - 128), c)
    return (signed(a) - signed(b)).abs()


def repaired_below(inter, top_k):
    """The magnitude, in e4m3 code units, from which the tiled gate/up GEMM on the e4m3 matrix core repairs
    the codes of h by default (default_requant_significance in csrc/moe_common.hpp): 128 at inter * top_k >= 16384,
    halved for every factor of four fewer terms per output, at least 8."""
    s, terms = 7, inter * top_k
    while terms < 16384 and s > 3:
        s, terms = s - 1, terms * 4
    return float(1 << s)


def oracle_down(h_q, h_s, ids, w2_q, w2_s):
    """The oracle's down projection applied to given h codes/scales [T, k, I]."""
    T, k, I = h_q.shape
    y = torch.zeros(T, k, w2_q.shape[1])
    for e in torch.unique(ids).tolist():
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        y[tok, slot] = moe.dequantize_groups(h_q[tok, slot], h_s[tok, slot]) @ \
            moe.dequantize_blocks(w2_q[e], w2_s[e]).T
    return y


def settle_disputed_codes(hq, mid, w13_q, w13_s, w2_q, w2_s, top_k, small_below=0.0):
    """Where the kernel's h codes differ from the oracle's, a float64 evaluation of the two dot products
    decides: the kernel's code must be the correct rounding of that value, or the value must sit on the
    rounding boundary to within the noise of an fp32 summation (the oracle's own matmul then lands on either
    side by luck). Returns (number of such codes, the oracle's output recomputed with the kernel's codes
    at those places): an fp32 evaluation of the layer that the kernel has to match to the stated bound.

    small_below > 0 (the tiled gate/up GEMM on the e4m3 matrix core, which repairs only the elements whose
    scaled magnitude reaches that many code units): a differing code whose two magnitudes are both at most
    small_below is not adjudicated and NOT taken over into the returned output, so whatever it does to the
    layer's output counts as the kernel's error; it must be within two code steps (or 2^-6 code units).
    mid: the oracle's intermediates, with ``ids`` indexing w13_q / w2_q."""
    T, k, I = hq.shape
    table = torch.from_numpy(moe.e4m3_decode_table()).double()
    steps = code_steps(hq, mid['h_q'])
    disputed = torch.nonzero(steps > 0).tolist()
    x_dq = moe.dequantize_groups(mid['x_q'], mid['x_s']).double()
    settled = []
    for t, j, c in disputed:
        mine = table[int(hq.view(torch.uint8)[t, j, c]) & 0x7f].item()
        theirs = table[int(mid['h_q'].view(torch.uint8)[t, j, c]) & 0x7f].item()
        if max(mine, theirs) <= small_below:
            # (near zero, where the format's steps are 2^-9 of the scale, the matrix core's error is an absolute
            # one and may span several steps: 2^-6 code units are 3.5e-5 of the group's maximum)
            mine_signed = -mine if int(hq.view(torch.uint8)[t, j, c]) & 0x80 else mine
            theirs_signed = -theirs if int(mid['h_q'].view(torch.uint8)[t, j, c]) & 0x80 else theirs
            assert int(steps[t, j, c]) <= 2 or abs(mine_signed - theirs_signed) <= 2.0 ** -6, \
                f'h[{t},{j},{c}]: {mine_signed} against {theirs_signed}: more than two code steps'
            continue
        e = int(mid['ids'][t, j])
        rows = torch.stack([w13_q[e, c], w13_q[e, I + c]]).float().double()
        scales = torch.stack([w13_s[e, c // 128], w13_s[e, (I + c) // 128]]).double().repeat_interleave(128, 1)
        prods = x_dq[t][None] * rows * scales
        g, u = prods.sum(dim=1)
        cond = (prods.abs().sum(dim=1) / prods.sum(dim=1).abs()).sum().item()
        v = abs((g / (1 + torch.exp(-g)) * u / mid['h_s'][t, j, c // 128].double()).item())
        boundary = (mine + theirs) / 2
        correct = mine if abs(v - mine) <= abs(v - theirs) else theirs
        edge = 1e-6 * cond + 2e-6
        assert mine == correct or abs(v - boundary) <= edge * max(v, 2.0 ** -9), \
            f'h[{t},{j},{c}]: scaled value {v!r} got the code of {mine}, the oracle has {theirs} (edge {edge:.1e})'
        settled.append((t, j, c))
    patched_q = mid['h_q'].clone()
    for t, j, c in settled:
        patched_q[t, j, c] = hq[t, j, c]
    y = mid['y'].clone()
    for t, j in sorted({(t, j) for t, j, _ in settled}):
        e = int(mid['ids'][t, j])
        y[t, j] = (moe.dequantize_groups(patched_q[t, j][None], mid['h_s'][t, j][None]) @
                   moe.dequantize_blocks(w2_q[e], w2_s[e]).T)[0]
    out = torch.zeros(T, y.shape[2])
    for j in range(top_k):
        out += mid['weights'][:, j:j + 1] * y[:, j]
    return len(settled), out
