"""Top-k selection of index scores on the GPU against the oracle, through the C ABI.
Integer work: the chosen indices and their order must be bit-exact."""
import pytest
import torch

from oracle import mla

pytestmark = pytest.mark.gpu


def run_kernel(capi, dev, scores, k, lengths=None):
    out = torch.full((scores.shape[0], k), -7, dtype=torch.int32, device=dev)
    capi.topk_select_launch(out, scores.to(dev), None if lengths is None else lengths.to(dev))
    torch.cuda.synchronize()
    return out.cpu()


@pytest.mark.parametrize('shape', [(3, 300, 40), (2, 32768, 2048), (5, 1000, 1000), (1, 5000, 1), (4, 70, 128),
                                   (2, 1024, 512), (3, 1025, 7), (2, 100000, 2048)])
def test_random_scores(capi, dev, shape):
    B, n, k = shape
    gen = torch.Generator().manual_seed(n + k)
    scores = torch.randn(B, n, generator=gen) * 3
    assert torch.equal(run_kernel(capi, dev, scores, k), mla.topk_select(scores, k))


def test_ties_specials_and_lengths(capi, dev):
    gen = torch.Generator().manual_seed(41)
    scores = torch.randint(-3, 4, (8, 3000), generator=gen).float()      # seven distinct values: ties everywhere
    scores[0, 5] = float('inf')
    scores[1, 7::11] = float('-inf')
    scores[2, 3::7] = float('nan')
    scores[3, ::2] = -0.0
    scores[3, 1::2] = 0.0
    scores[4] = 1.5                                                      # one value only
    scores[5] = float('nan')
    lengths = torch.tensor([3000, 2999, 1024, 1023, 1, 17, 0, 5000], dtype=torch.int32)
    for k in (1, 64, 1024, 2048, 3000, 3100):
        for ln in (None, lengths):
            got = run_kernel(capi, dev, scores, k, ln)
            assert torch.equal(got, mla.topk_select(scores, k, ln)), (k, ln is not None)


def test_denormals_and_close_values(capi, dev):
    # keys that differ only in the last byte, across zero
    base = torch.tensor([1e-42, -1e-42, 0.0, 1.0, 1.0 + 2 ** -23, 1.0 - 2 ** -24, -1.0, 3e38, -3e38])
    gen = torch.Generator().manual_seed(42)
    scores = base[torch.randint(0, base.numel(), (4, 4096), generator=gen)]
    for k in (1, 100, 2048, 4096):
        assert torch.equal(run_kernel(capi, dev, scores, k), mla.topk_select(scores, k))


def test_selected_indices_feed_the_attention(capi, dev):
    # selection -> sparse-MLA decode; shorter requests leave -1 entries, which the attention skips
    gen = torch.Generator().manual_seed(43)
    B, H, N, k = 3, 128, 1024, 256
    q, kv, _ = mla.mla_make_inputs(B, H, N, k, generator=gen)
    scores = torch.randn(B, N, generator=gen)
    lengths = torch.tensor([1024, 100, 300], dtype=torch.int32)
    idx = torch.empty(B, k, dtype=torch.int32, device=dev)
    capi.topk_select_launch(idx, scores.to(dev), lengths.to(dev))
    out = torch.empty(B, H, 512, dtype=torch.float32, device=dev)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, k), dtype=torch.uint8, device=dev)
    capi.sparse_mla_decode_launch(out, q.to(dev), kv.to(dev), idx, ws)
    torch.cuda.synchronize()
    want_idx = mla.topk_select(scores, k, lengths)
    assert torch.equal(idx.cpu(), want_idx) and (want_idx[1] == -1).sum() == k - 100
    ref = mla.sparse_mla_decode(q, kv, want_idx, out_dtype=torch.float32)
    assert mla.rel_rms_error(out.cpu(), ref) <= 2e-2


def test_rejects_bad_arguments(capi, dev):
    with pytest.raises(ValueError):
        capi.topk_select_launch(torch.zeros(2, 4, dtype=torch.int32, device=dev),
                                torch.zeros(2, 8, dtype=torch.float64, device=dev))
