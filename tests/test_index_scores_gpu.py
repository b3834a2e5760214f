"""Indexer scores on the GPU against the oracle, through the C ABI.

bf16 products are exact in fp32, so the kernel differs from a float64 evaluation only by fp32 accumulation over
the 128 dimensions and the heads: |err| <= 192 * 2^-24 * sum_h |w_h| * scale * (|q_h| . |k_t|), far below anything
that moves the selection except on near-ties. Positions at or beyond a request's length must be -inf exactly."""
import pytest
import torch

from oracle import mla

pytestmark = pytest.mark.gpu


def make(B, Hi, N, seed, dev=None):
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hi, 128, generator=gen).bfloat16()
    k = torch.randn(B, N, 128, generator=gen).bfloat16()
    w = torch.randn(B, Hi, generator=gen) * Hi ** -0.5
    return q, k, w


def run_kernel(capi, dev, q, k, w, lengths=None, scale=128 ** -0.5):
    scores = torch.full((q.shape[0], k.shape[1]), float('nan'), device=dev)
    capi.mla_index_scores_launch(scores, q.to(dev), k.to(dev), w.to(dev), None if lengths is None else lengths.to(dev),
                                 scale)
    torch.cuda.synchronize()
    return scores.cpu()


def check(got, q, k, w, lengths, scale=128 ** -0.5):
    s = torch.einsum('bhd,bnd->bhn', q.double(), k.double()) * scale
    want = torch.einsum('bh,bhn->bn', w.double(), torch.relu(s))
    bound = 192 * 2.0 ** -24 * torch.einsum('bh,bhn->bn', w.double().abs(),
                                           torch.einsum('bhd,bnd->bhn', q.double().abs(), k.double().abs()) * scale)
    N = k.shape[1]
    live = torch.ones(q.shape[0], N, dtype=torch.bool) if lengths is None else \
        torch.arange(N)[None, :] < lengths[:, None].long()
    assert ((got.double() - want).abs()[live] <= bound[live] + 1e-12).all()
    assert (got[~live] == float('-inf')).all()


@pytest.mark.parametrize('shape', [(2, 64, 512), (3, 32, 100), (1, 64, 33), (2, 64, 1025), (4, 32, 2048), (1, 64, 1),
                                   (2, 64, 4096 + 17)])
def test_matches_float64(capi, dev, shape):
    B, Hi, N = shape
    q, k, w = make(B, Hi, N, B * 100 + N)
    check(run_kernel(capi, dev, q, k, w), q, k, w, None)
    lengths = torch.randint(0, N + 1, (B,), generator=torch.Generator().manual_seed(N)).int()
    lengths[0] = N
    got = run_kernel(capi, dev, q, k, w, lengths, 0.3)
    check(got, q, k, w, lengths, 0.3)
    # as close to the exact scores as the oracle's own fp32 evaluation
    torch.testing.assert_close(got, mla.index_scores(q, k, w, lengths, 0.3), rtol=1e-4, atol=1e-5)


def test_golden_fixture_inputs(capi, dev):
    import numpy as np
    from pathlib import Path
    z = np.load(Path(__file__).parent / 'golden' / 'indexer_golden.npz')
    q, k, w = torch.from_numpy(z['q']).bfloat16(), torch.from_numpy(z['k']).bfloat16(), torch.from_numpy(z['w'])
    scale = float(z['scale'][0])
    got = run_kernel(capi, dev, q, k, w, None, scale)
    check(got, q, k, w, None, scale)
    # the selection from the kernel's scores is the one the oracle makes from its scores of the same bf16 inputs
    want = mla.topk_select(mla.index_scores(q, k, w, None, scale), z['topk'].shape[1])
    idx = torch.empty_like(want, device=dev)
    capi.topk_select_launch(idx, got.to(dev))
    torch.cuda.synchronize()
    assert (idx.cpu() != want).any(dim=1).sum().item() == 0


def test_scores_selection_attention_chain(capi, dev):
    # one decode step of sparse attention: scores -> top-k -> gather/attend, against the oracle's chain
    B, H, Hi, N, topk = 3, 128, 64, 4096, 512
    q_idx, k_idx, w = make(B, Hi, N, 7)
    gen = torch.Generator().manual_seed(8)
    q, kv, _ = mla.mla_make_inputs(B, H, N, topk, generator=gen)
    lengths = torch.tensor([N, 3000, 700], dtype=torch.int32)
    scores = torch.empty(B, N, device=dev)
    idx = torch.empty(B, topk, dtype=torch.int32, device=dev)
    out = torch.empty(B, H, 512, device=dev)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, topk), dtype=torch.uint8, device=dev)
    capi.mla_index_scores_launch(scores, q_idx.to(dev), k_idx.to(dev), w.to(dev), lengths.to(dev))
    capi.topk_select_launch(idx, scores, lengths.to(dev))
    capi.sparse_mla_decode_launch(out, q.to(dev), kv.to(dev), idx, ws)
    torch.cuda.synchronize()
    want_idx = mla.topk_select(mla.index_scores(q_idx, k_idx, w, lengths), topk, lengths)
    differing = (idx.cpu() != want_idx).any(dim=1).sum().item()
    assert differing == 0            # (a near-tie at the 512th score could flip one entry; none at this seed)
    ref = mla.sparse_mla_decode(q, kv, want_idx, out_dtype=torch.float32)
    assert mla.rel_rms_error(out.cpu(), ref) <= 2e-2


def test_full_workload_shape(capi, dev):
    B, Hi, N = 64, 64, 32768
    gen = torch.Generator(device=dev).manual_seed(20262)
    q = torch.randn(B, Hi, 128, device=dev, generator=gen).bfloat16()
    k = torch.randn(B, N, 128, device=dev, generator=gen).bfloat16()
    w = torch.randn(B, Hi, device=dev, generator=gen) / 8
    scores = torch.empty(B, N, device=dev)
    capi.mla_index_scores_launch(scores, q, k, w)
    torch.cuda.synchronize()
    for b0 in range(0, B, 16):                      # the oracle's [16, 64, 32768] fp32 intermediate is 134 MB
        want = mla.index_scores(q[b0:b0 + 16], k[b0:b0 + 16], w[b0:b0 + 16])
        torch.testing.assert_close(scores[b0:b0 + 16], want, rtol=1e-4, atol=1e-4)


def test_rejects_unsupported_shapes(capi, dev):
    q, k, w = make(1, 48, 64, 1)
    with pytest.raises(capi.LaunchRejected):
        run_kernel(capi, dev, q, k, w)


def test_paged_key_cache(capi, dev):
    # the pages of a contiguous cache scattered into a pool: the same scores, bit for bit, on mapped pages;
    # -inf on an unmapped page and beyond the lengths; then the whole paged chain scores -> selection -> attention
    gen = torch.Generator().manual_seed(11)
    B, H, Hi, N, page, topk = 3, 128, 64, 1024, 64, 200
    q_idx, k_idx, w = make(B, Hi, N, 12)
    q, kv, _ = mla.mla_make_inputs(B, H, N, topk, generator=gen)
    k_pool, table = mla.mla_scatter_into_pool(k_idx, page, generator=gen)
    kv_pool = torch.randn(k_pool.shape[0], page, 576, generator=gen).bfloat16()
    kv_pool[table.reshape(-1).long()] = kv.reshape(-1, page, 576)            # the latent cache shares the block table
    lengths = torch.tensor([N, 700, 333], dtype=torch.int32)
    want = run_kernel(capi, dev, q_idx, k_idx, w, lengths)
    table[1, 2] = -1
    want[1, 128:192] = float('-inf')
    scores = torch.full((B, N), float('nan'), device=dev)
    capi.mla_index_scores_paged_launch(scores, q_idx.to(dev), k_pool.to(dev), table.to(dev), w.to(dev), lengths.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(scores.cpu(), want)
    idx = torch.empty(B, topk, dtype=torch.int32, device=dev)
    out = torch.empty(B, H, 512, device=dev)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, topk), dtype=torch.uint8, device=dev)
    capi.topk_select_launch(idx, scores, lengths.to(dev))
    capi.sparse_mla_decode_paged_launch(out, q.to(dev), kv_pool.to(dev), table.to(dev), idx, ws)
    torch.cuda.synchronize()
    want_idx = mla.topk_select(want, topk, lengths)
    assert torch.equal(idx.cpu(), want_idx)
    ref = mla.sparse_mla_decode_paged(q, kv_pool, table, want_idx, out_dtype=torch.float32)
    assert mla.rel_rms_error(out.cpu(), ref) <= 2e-2
