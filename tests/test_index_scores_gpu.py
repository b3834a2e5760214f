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


# ---- e4m3 index keys -----------------------------------------------------------------------------------------
# The products of e4m3 codes are exact, but the matrix core adds the 64 products of a step with about 16
# significant bits (measured on gfx950: up to 2^-16 of the sum of |products| per step), so the bound against
# float64 is 2^-13 * k_scale * sum_h |w_h| * scale * (|q_h| . |k_t|) instead of the 192 * 2^-24 of the bf16 form.

def make_fp8(B, Hi, N, seed):
    from oracle import moe
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hi, 128, generator=gen)
    k = torch.randn(B, N, 128, generator=gen) * (0.5 + torch.rand(B, N, 1, generator=gen) * 4)
    w = torch.randn(B, Hi, generator=gen) * Hi ** -0.5
    qq, qs = moe.quantize_groups(q.reshape(B * Hi, 128))
    kq, ks = moe.quantize_groups(k.reshape(B * N, 128))
    return (qq.view(torch.uint8).reshape(B, Hi, 128), kq.view(torch.uint8).reshape(B, N, 128), ks.reshape(B, N).contiguous(),
            (w * qs.reshape(B, Hi)).contiguous())


def run_fp8(capi, dev, qc, kc, ks, w, lengths=None, scale=128 ** -0.5):
    scores = torch.full((qc.shape[0], kc.shape[1]), float('nan'), device=dev)
    capi.mla_index_scores_fp8_launch(scores, qc.to(dev), kc.to(dev), ks.to(dev), w.to(dev),
                                     None if lengths is None else lengths.to(dev), scale)
    torch.cuda.synchronize()
    return scores.cpu()


def check_fp8(got, qc, kc, ks, w, lengths, scale=128 ** -0.5):
    q, k = mla.e4m3_to_float(qc).double(), mla.e4m3_to_float(kc).double()
    want = mla.index_scores_fp8(qc, kc, ks, w, None, scale).double()
    bound = 2.0 ** -13 * ks.double() * torch.einsum('bh,bhn->bn', w.double().abs(),
                                                    torch.einsum('bhd,bnd->bhn', q.abs(), k.abs()) * scale)
    N = kc.shape[1]
    live = torch.ones(qc.shape[0], N, dtype=torch.bool) if lengths is None else \
        torch.arange(N)[None, :] < lengths[:, None].long()
    assert ((got.double() - want).abs()[live] <= bound[live] + 1e-12).all()
    assert (got[~live] == float('-inf')).all()


@pytest.mark.parametrize('shape', [(2, 64, 512), (3, 32, 100), (1, 64, 33), (2, 64, 1025), (4, 32, 2048), (1, 64, 1),
                                   (2, 64, 4096 + 17)])
def test_fp8_matches_float64(capi, dev, shape):
    B, Hi, N = shape
    qc, kc, ks, w = make_fp8(B, Hi, N, B * 100 + N)
    check_fp8(run_fp8(capi, dev, qc, kc, ks, w), qc, kc, ks, w, None)
    lengths = torch.randint(0, N + 1, (B,), generator=torch.Generator().manual_seed(N)).int()
    lengths[0] = N
    check_fp8(run_fp8(capi, dev, qc, kc, ks, w, lengths, 0.3), qc, kc, ks, w, lengths, 0.3)


def test_fp8_exact_on_small_integers(capi, dev):
    # codes of small integers and power-of-two scales: every product and every sum is exact in any order
    gen = torch.Generator().manual_seed(5)
    B, Hi, N = 2, 64, 300
    q = torch.randint(-2, 3, (B, Hi, 128), generator=gen).float()
    k = torch.randint(-2, 3, (B, N, 128), generator=gen).float()
    qc, kc = q.to(torch.float8_e4m3fn).view(torch.uint8), k.to(torch.float8_e4m3fn).view(torch.uint8)
    ks = torch.pow(2.0, torch.randint(-3, 4, (B, N), generator=gen).float())
    w = torch.randint(-4, 5, (B, Hi), generator=gen).float() / 8
    got = run_fp8(capi, dev, qc, kc, ks, w, None, 0.25)
    assert torch.equal(got, mla.index_scores_fp8(qc, kc, ks, w, None, 0.25))


def test_fp8_keys_from_the_quantiser_and_selection(capi, dev):
    # the caller's chain: bf16 keys -> per-row e4m3 quantiser -> scores -> top-k, against the oracle on the same codes
    gen = torch.Generator().manual_seed(21)
    B, Hi, N, topk = 2, 64, 2048, 256
    qc, _, _, w = make_fp8(B, Hi, N, 22)
    k = (torch.randn(B, N, 128, generator=gen) * 3).bfloat16()
    codes = torch.empty(B * N, 128, dtype=torch.uint8, device=dev)
    scales = torch.empty(B * N, 1, device=dev)
    capi.moe_quant_bf16_launch(codes, scales, k.reshape(B * N, 128).to(dev))
    scores = torch.empty(B, N, device=dev)
    capi.mla_index_scores_fp8_launch(scores, qc.to(dev), codes.view(B, N, 128), scales.view(B, N), w.to(dev))
    idx = torch.empty(B, topk, dtype=torch.int32, device=dev)
    capi.topk_select_launch(idx, scores)
    torch.cuda.synchronize()
    check_fp8(scores.cpu(), qc, codes.cpu().view(B, N, 128), scales.cpu().view(B, N), w, None)
    assert torch.equal(idx.cpu(), mla.topk_select(scores.cpu(), topk))
    # against the selection from the unquantised keys: the quantisation moves a few entries near the boundary only
    exact = mla.topk_select(mla.index_scores(mla.e4m3_to_float(qc).bfloat16(), k, w), topk)
    overlap = sum(len(set(idx[b].tolist()) & set(exact[b].tolist())) for b in range(B)) / (B * topk)
    assert overlap > 0.9


@pytest.mark.parametrize('page', [16, 64, 256])
def test_fp8_paged_key_cache(capi, dev, page):
    gen = torch.Generator().manual_seed(31 + page)
    B, Hi, N = 3, 64, 1024
    qc, kc, ks, w = make_fp8(B, Hi, N, 32)
    lengths = torch.tensor([N, 700, 333], dtype=torch.int32)
    want = run_fp8(capi, dev, qc, kc, ks, w, lengths)
    per_req = N // page
    n_pages = B * per_req + 3
    order = torch.randperm(n_pages, generator=gen)[:B * per_req]
    k_pool = torch.randint(0, 0x7f, (n_pages, page, 128), generator=gen).to(torch.uint8)
    s_pool = torch.rand(n_pages, page, generator=gen)
    k_pool[order] = kc.reshape(B * per_req, page, 128)
    s_pool[order] = ks.reshape(B * per_req, page)
    table = order.reshape(B, per_req).int()
    table[1, 2] = -1
    want[1, 2 * page:3 * page] = float('-inf')
    scores = torch.full((B, N), float('nan'), device=dev)
    capi.mla_index_scores_fp8_paged_launch(scores, qc.to(dev), k_pool.to(dev), s_pool.to(dev), table.to(dev), w.to(dev),
                                           lengths.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(scores.cpu(), want)


def test_fp8_full_workload_shape(capi, dev):
    B, Hi, N = 64, 64, 32768
    gen = torch.Generator(device=dev).manual_seed(20263)
    qc = torch.randn(B, Hi, 128, device=dev, generator=gen).to(torch.float8_e4m3fn).view(torch.uint8)
    kc = torch.randn(B, N, 128, device=dev, generator=gen).to(torch.float8_e4m3fn).view(torch.uint8)
    ks = torch.rand(B, N, device=dev, generator=gen) + 0.5
    w = torch.randn(B, Hi, device=dev, generator=gen) / 8
    scores = torch.empty(B, N, device=dev)
    capi.mla_index_scores_fp8_launch(scores, qc, kc, ks, w)
    torch.cuda.synchronize()
    for b0 in range(0, B, 16):                      # the oracle's float64 intermediate of 16 requests is 268 MB
        want = mla.index_scores_fp8(qc[b0:b0 + 16], kc[b0:b0 + 16], ks[b0:b0 + 16], w[b0:b0 + 16])
        torch.testing.assert_close(scores[b0:b0 + 16], want, rtol=2e-3, atol=2e-3)


def test_fp8_rejects_unsupported_shapes(capi, dev):
    qc, kc, ks, w = make_fp8(1, 48, 64, 1)
    with pytest.raises(capi.LaunchRejected):
        run_fp8(capi, dev, qc, kc, ks, w)
