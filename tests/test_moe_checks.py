"""CPU tests of the checker the GPU parity tests of the MoE layer lean on: settle_disputed_codes accepts a
differing code of h only when a float64 evaluation puts the value on the rounding boundary to within fp32
summation noise, and refuses any other difference."""
import pytest
import torch

from oracle import moe

from moe_checks import code_steps, repaired_below, settle_disputed_codes


def tiny_layer(seed=3):
    gen = torch.Generator().manual_seed(seed)
    E, H, I, T, k = 3, 256, 128, 24, 2
    w = moe.moe_make_weights(E, H, I, gen)
    x, logits = moe.moe_make_inputs(T, H, E, gen)
    ref, mid = moe.moe_forward(x, logits, *w, top_k=k, out_dtype=torch.float32, return_intermediates=True)
    return w, ref, mid, k


def neighbour(code, up):
    """The e4m3 code one step further from (up) or closer to zero."""
    c = int(code)
    return (c + 1) if up else (c - 1)


def test_identical_codes_settle_to_the_oracle_output():
    w, ref, mid, k = tiny_layer()
    n, out = settle_disputed_codes(mid['h_q'].clone(), mid, *w, k)
    assert n == 0 and torch.equal(out, ref)


def test_a_code_flipped_far_from_a_boundary_is_refused():
    w, ref, mid, k = tiny_layer()
    table = torch.from_numpy(moe.e4m3_decode_table()).double()
    raw = mid['h_q'].view(torch.uint8)
    # an element in the middle of its code's interval: take a mid-range code and move it one step
    mags = raw & 0x7f
    t, j, c = [int(v) for v in torch.nonzero((mags > 0x40) & (mags < 0x7e))[0]]
    x_dq = moe.dequantize_groups(mid['x_q'], mid['x_s']).double()
    flipped = mid['h_q'].clone()
    flipped.view(torch.uint8)[t, j, c] = neighbour(raw[t, j, c], up=True)
    # (make sure the pick is not itself a boundary case: the exact value is nearer to the oracle's code)
    e = int(mid['ids'][t, j])
    I = mid['h_q'].shape[2]
    g = (x_dq[t] * moe.dequantize_blocks(w[0][e], w[1][e]).double()[c]).sum()
    u = (x_dq[t] * moe.dequantize_blocks(w[0][e], w[1][e]).double()[I + c]).sum()
    v = abs((g / (1 + torch.exp(-g)) * u / mid['h_s'][t, j, c // 128].double()).item())
    mine, theirs = table[int(flipped.view(torch.uint8)[t, j, c]) & 0x7f].item(), table[int(raw[t, j, c]) & 0x7f].item()
    assert abs(v - theirs) < 0.45 * abs(mine - theirs)
    with pytest.raises(AssertionError, match='got the code of'):
        settle_disputed_codes(flipped, mid, *w, k)


def test_a_code_on_the_boundary_is_settled_and_changes_the_reference():
    """An oracle whose scale is nudged so that one element's scaled value sits exactly between two codes: either
    code is then acceptable, and the returned output carries the kernel's choice."""
    w, ref, mid, k = tiny_layer()
    table = torch.from_numpy(moe.e4m3_decode_table()).double()
    raw = mid['h_q'].view(torch.uint8)
    mags = raw & 0x7f
    t, j, c = [int(v) for v in torch.nonzero((mags > 0x40) & (mags < 0x7e))[0]]
    e, I = int(mid['ids'][t, j]), mid['h_q'].shape[2]
    x_dq = moe.dequantize_groups(mid['x_q'], mid['x_s']).double()
    wd = moe.dequantize_blocks(w[0][e], w[1][e]).double()
    g, u = (x_dq[t] * wd[c]).sum(), (x_dq[t] * wd[I + c]).sum()
    h = abs((g / (1 + torch.exp(-g)) * u).item())
    here, above = table[int(mags[t, j, c])].item(), table[int(mags[t, j, c]) + 1].item()
    mid = dict(mid, h_s=mid['h_s'].clone())
    mid['h_s'][t, j, c // 128] = h / ((here + above) / 2)           # the value now sits on the boundary
    flipped = mid['h_q'].clone()
    flipped.view(torch.uint8)[t, j, c] = neighbour(raw[t, j, c], up=True)
    n, out = settle_disputed_codes(flipped, mid, *w, k)
    assert n == 1
    assert (out[t] - ref[t]).abs().max() > 0 and torch.equal(out[:t], ref[:t]) and torch.equal(out[t + 1:], ref[t + 1:])


def test_small_codes_are_tolerated_but_not_settled():
    w, ref, mid, k = tiny_layer()
    raw = mid['h_q'].view(torch.uint8)
    mags = raw & 0x7f
    small = torch.nonzero((mags > 0x20) & (mags < 0x50))               # well below 64 code units
    large = torch.nonzero((mags > 0x72) & (mags < 0x7e))               # above 128
    flipped = mid['h_q'].clone()
    t, j, c = [int(v) for v in small[0]]
    flipped.view(torch.uint8)[t, j, c] = neighbour(raw[t, j, c], up=False)
    n, out = settle_disputed_codes(flipped, mid, *w, k, small_below=64.0)
    assert n == 0 and torch.equal(out, ref)                            # tolerated, and its effect stays an error
    with pytest.raises(AssertionError):
        settle_disputed_codes(flipped, mid, *w, k)                     # the exact forms get no such allowance
    t, j, c = [int(v) for v in large[0]]
    flipped = mid['h_q'].clone()
    flipped.view(torch.uint8)[t, j, c] = neighbour(raw[t, j, c], up=False)
    with pytest.raises(AssertionError):
        settle_disputed_codes(flipped, mid, *w, k, small_below=64.0)   # a large code is held to the exact rule
    far = mid['h_q'].clone()
    t, j, c = [int(v) for v in small[0]]
    far.view(torch.uint8)[t, j, c] = int(raw[t, j, c]) - 3
    with pytest.raises(AssertionError, match='more than two code steps'):
        settle_disputed_codes(far, mid, *w, k, small_below=64.0)


def test_code_steps_and_threshold():
    a = torch.tensor([0x00, 0x80, 0x01, 0x81, 0x7e], dtype=torch.uint8).view(torch.float8_e4m3fn)
    b = torch.tensor([0x80, 0x00, 0x81, 0x01, 0x7d], dtype=torch.uint8).view(torch.float8_e4m3fn)
    assert code_steps(a, b).tolist() == [0, 0, 2, 2, 1]
    assert [repaired_below(i, k) for i, k in ((2048, 8), (2048, 2), (256, 2), (128, 1), (8192, 8))] == \
        [128.0, 64.0, 16.0, 8.0, 128.0]
