"""The entry point that allocates nothing (sparse_mla_decode_static_launcher): through the C ABI, against
sparse_mla_decode_launcher on the same inputs, bit for bit; two calls in a row, the second on a smaller problem,
so that what the first call left in the library's static scratch array is in the way of the second."""
import pytest
import torch

from oracle import mla

pytestmark = pytest.mark.gpu


def both_ways(capi, dev, B, H, N, topk, seed, dtype):
    gen = torch.Generator().manual_seed(seed)
    q, kv, idx = (t.to(dev) for t in mla.mla_make_inputs(B, H, N, topk, generator=gen))
    want = torch.full((B, H, 512), float('nan'), dtype=dtype, device=dev)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, topk), dtype=torch.uint8, device=dev)
    capi.sparse_mla_decode_launch(want, q, kv, idx, ws)
    got = torch.full((B, H, 512), float('nan'), dtype=dtype, device=dev)
    # a first call may look up the array's address; the call that is watched comes after it. What is watched is the
    # driver's count of free device memory (an allocation inside the library would not show in torch's allocator).
    capi.sparse_mla_decode_static_launch(got, q, kv, idx)
    torch.cuda.synchronize()
    got.fill_(float('nan'))
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(dev), torch.cuda.mem_get_info(dev)[0]
    capi.sparse_mla_decode_static_launch(got, q, kv, idx)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    return got, want, (q, kv, idx)


def test_static_scratch_entry_point_matches_the_workspace_one(capi, dev):
    assert capi.library().sparse_mla_decode_static_scratch_bytes() == 72 << 20
    # the workload's request shape: 128 heads, 2048 selected rows, 4 key splits per request
    got, want, ins = both_ways(capi, dev, 8, 128, 4096, 2048, 5, torch.float32)
    assert torch.isfinite(want).all() and torch.equal(got, want)
    ref = mla.sparse_mla_decode(*(t.cpu() for t in ins), out_dtype=torch.float32)
    assert mla.rel_rms_error(got.cpu(), ref) <= 2e-2
    # a smaller problem right behind it (other split count, other head kernel): stale partials must not show
    got, want, _ = both_ways(capi, dev, 3, 64, 700, 100, 6, torch.bfloat16)
    assert torch.isfinite(want.float()).all() and torch.equal(got, want)
    got, want, _ = both_ways(capi, dev, 1, 128, 300, 33, 7, torch.bfloat16)
    assert torch.equal(got, want)


def test_static_scratch_entry_point_rejects_what_does_not_fit(capi, dev):
    B, H, topk = 80, 128, 2048          # 80 requests x 4 splits need 84 213 760 bytes
    assert capi.sparse_mla_workspace_bytes(B, H, topk) > capi.library().sparse_mla_decode_static_scratch_bytes()
    q = torch.zeros(B, H, 576, dtype=torch.bfloat16, device=dev)
    kv = torch.zeros(B, 2048, 576, dtype=torch.bfloat16, device=dev)
    idx = torch.zeros(B, topk, dtype=torch.int32, device=dev)
    out = torch.full((B, H, 512), 7.0, dtype=torch.bfloat16, device=dev)
    with pytest.raises(capi.LaunchRejected, match='static array'):
        capi.sparse_mla_decode_static_launch(out, q, kv, idx)
    torch.cuda.synchronize()
    assert (out == 7.0).all()           # nothing was launched
