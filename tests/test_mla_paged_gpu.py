"""Sparse-MLA decode over a paged cache, through the C ABI.

The paged launcher runs the same kernels as the contiguous one and differs only in how a selected
key becomes a row address, so the bar is bit-equality: a pool that holds the pages of a contiguous
cache at permuted page numbers must give exactly the contiguous launcher's output, with and
without a block table. Padding rules (negative keys, positions beyond the table, unmapped pages,
rows beyond the pool) are checked against the oracle's resolution of the same table, to the
operator's bound (max |out - ref| <= 2e-2 rms(ref) on the fp32 output)."""
import pytest
import torch

from oracle import mla

pytestmark = pytest.mark.gpu
TOL = 2e-2


def run_contiguous(capi, q, kv, idx, config=0, dtype=torch.bfloat16):
    B, H, _ = q.shape
    out = torch.full((B, H, 512), float('nan'), device=q.device, dtype=dtype)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, idx.shape[1], config), dtype=torch.uint8,
                     device=q.device)
    capi.sparse_mla_decode_launch(out, q, kv, idx, ws, config=config)
    torch.cuda.synchronize()
    return out


def run_paged(capi, q, pool, table, idx, config=0, dtype=torch.bfloat16):
    B, H, _ = q.shape
    out = torch.full((B, H, 512), float('nan'), device=q.device, dtype=dtype)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, idx.shape[1], config), dtype=torch.uint8,
                     device=q.device)
    capi.sparse_mla_decode_paged_launch(out, q, pool, table, idx, ws, config=config)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize('config', [0, 3, 1002])
@pytest.mark.parametrize('shape', [(2, 128, 512, 300, 64), (3, 32, 96, 33, 16), (1, 64, 512, 257, 64),
                                   (2, 128, 4096, 2048, 64), (1, 256, 256, 64, 128), (4, 128, 64, 1, 1)])
def test_paged_is_bit_equal_to_contiguous(capi, dev, shape, config):
    B, H, N, topk, page = shape
    gen = torch.Generator().manual_seed(B * 1000 + topk + page)
    q, kv, idx = mla.mla_make_inputs(B, H, N, topk, generator=gen)
    if topk > 4:
        idx[0, 2] = -1
        idx[-1, topk - 1] = N + 5
    pool, table = mla.mla_scatter_into_pool(kv, page, generator=gen)
    rows = mla.resolve_paged_indices(idx, table, page, pool.shape[0] * page).int()
    q, kv, idx, pool, table, rows = (t.to(dev) for t in (q, kv, idx, pool, table, rows))
    for dtype in (torch.bfloat16, torch.float32):
        want = run_contiguous(capi, q, kv, idx, config, dtype)
        assert torch.isfinite(want).all()
        assert torch.equal(run_paged(capi, q, pool, table, idx, config, dtype), want)
        assert torch.equal(run_paged(capi, q, pool, None, rows, config, dtype), want)


def test_padding_rules_of_the_block_table(capi, dev):
    gen = torch.Generator().manual_seed(11)
    B, H, N, topk, page = 3, 128, 1024, 400, 64
    q, kv, idx = mla.mla_make_inputs(B, H, N, topk, generator=gen)
    pool, table = mla.mla_scatter_into_pool(kv, page, generator=gen)
    table[0, 3] = -1                       # an unmapped page
    table[1, 5] = pool.shape[0] + 7        # a page beyond the pool
    table = table[:, :12].contiguous()     # positions >= 768 are beyond the table
    idx[2, :5] = torch.tensor([-1, -7, 2 ** 31 - 1, 768, 767])
    q, pool, table, idx = (t.to(dev) for t in (q, pool, table, idx))
    rows = mla.resolve_paged_indices(idx, table, page, pool.shape[0] * page)
    assert (rows < 0).sum() > 100 and (rows >= 0).sum() > 100
    ref = mla.sparse_mla_decode_paged(q, pool, table, idx, out_dtype=torch.float32)
    got = run_paged(capi, q, pool, table, idx, 0, torch.float32)
    assert torch.isfinite(got).all()
    assert mla.rel_rms_error(got, ref) <= TOL
    # dropping the padded selections by hand gives the same bits
    assert torch.equal(run_paged(capi, q, pool, None, rows.int(), 0, torch.float32), got)


def test_requests_may_share_pages(capi, dev):
    # a common prefix: two requests map their first logical pages to the same physical pages
    gen = torch.Generator().manual_seed(12)
    B, H, N, topk, page = 2, 128, 512, 256, 64
    q, kv, idx = mla.mla_make_inputs(B, H, N, topk, generator=gen)
    kv[1, :256] = kv[0, :256]
    pool, table = mla.mla_scatter_into_pool(kv, page, generator=gen)
    table[1, :4] = table[0, :4]
    q, kv, idx, pool, table = (t.to(dev) for t in (q, kv, idx, pool, table))
    assert torch.equal(run_paged(capi, q, pool, table, idx), run_contiguous(capi, q, kv, idx))


def test_full_workload_shape_paged(capi, dev):
    # the benchmark's shape with the cache held as 64-row pages: 64 x 512 pages of one pool
    gen = torch.Generator(device=dev).manual_seed(20253)
    B, H, N, topk, page = 64, 128, 32768, 2048, 64
    q, kv, idx = mla.mla_make_inputs(B, H, N, topk, generator=gen, device=dev)
    per_req = N // page
    order = torch.randperm(B * per_req, generator=gen, device=dev)
    pool = torch.empty(B * per_req, page, 576, dtype=torch.bfloat16, device=dev)
    pool[order] = kv.reshape(B * per_req, page, 576)
    table = order.reshape(B, per_req).int()
    want = run_contiguous(capi, q, kv, idx)
    assert torch.equal(run_paged(capi, q, pool, table, idx), want)


def test_rejects_bad_page_geometry(capi, dev):
    q = torch.zeros(1, 128, 576, dtype=torch.bfloat16, device=dev)
    idx = torch.zeros(1, 32, dtype=torch.int32, device=dev)
    table = torch.zeros(1, 4, dtype=torch.int32, device=dev)
    out = torch.zeros(1, 128, 512, dtype=torch.bfloat16, device=dev)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(1, 128, 32, 0), dtype=torch.uint8, device=dev)
    pool = torch.zeros(4, 48, 576, dtype=torch.bfloat16, device=dev)      # page size not a power of two
    with pytest.raises(capi.LaunchRejected):
        capi.sparse_mla_decode_paged_launch(out, q, pool, table, idx, ws)
    pool = torch.zeros(4, 64, 576, dtype=torch.bfloat16, device=dev)
    with pytest.raises(capi.LaunchRejected):
        capi.sparse_mla_decode_paged_launch(out, q, pool, table, idx, ws[:16])
    torch.cuda.synchronize()
