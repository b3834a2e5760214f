"""The e4m3 storage form of the latent cache on the GPU, through the C ABI: the quantiser that writes it
(bit-exact against the oracle's bytes) and sparse-MLA decode over it (bit-equal to the bf16 launcher on the
dequantised cache; max |out - ref| <= 2e-2 * rms(ref) against the fp32 oracle on the dequantised rows)."""
import pytest
import torch

from oracle import mla

pytestmark = pytest.mark.gpu
TOL = 2e-2


def make_cache(capi, dev, kv, config=0):
    cache = torch.empty(*kv.shape[:-1], 656, dtype=torch.uint8, device=dev)
    capi.mla_latent_quant_launch(cache, kv.to(dev), config)
    torch.cuda.synchronize()
    return cache


@pytest.mark.parametrize('config', [0, 32])
@pytest.mark.parametrize('rows', [1, 3, 257, 4096])
def test_quantiser_bytes(capi, dev, rows, config):
    gen = torch.Generator().manual_seed(rows + config)
    kv = (torch.randn(rows, 576, generator=gen) * torch.exp(torch.randn(rows, 1, generator=gen))).bfloat16()
    if rows > 2:
        kv[1, :128] = 0                       # a block of zeros: the floor scale, codes 0
        kv[2, 130] = 3.0e38                   # a huge value
    got = make_cache(capi, dev, kv, config).cpu()
    want = mla.latent_quantize(kv, pow2=config == 32)
    assert torch.equal(got, want)


def run_fp8(capi, dev, q, cache, idx, dtype=torch.bfloat16, config=0):
    B, H, _ = q.shape
    out = torch.full((B, H, 512), float('nan'), device=dev, dtype=dtype)
    ws = torch.empty(capi.sparse_mla_fp8_workspace_bytes(B, H, idx.shape[1], config), dtype=torch.uint8, device=dev)
    ws.fill_(0xff)                            # (padding rows of the compact block must not matter: NaN patterns)
    capi.sparse_mla_decode_fp8_launch(out, q.to(dev), cache, idx.to(dev), ws, config=config)
    torch.cuda.synchronize()
    return out.cpu()


def run_bf16(capi, dev, q, kv, idx, dtype=torch.bfloat16, config=0):
    B, H, _ = q.shape
    out = torch.full((B, H, 512), float('nan'), device=dev, dtype=dtype)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, idx.shape[1], config), dtype=torch.uint8, device=dev)
    capi.sparse_mla_decode_launch(out, q.to(dev), kv.to(dev), idx.to(dev), ws, config=config)
    torch.cuda.synchronize()
    return out.cpu()


@pytest.mark.parametrize('shape', [(2, 128, 512, 64), (3, 128, 4096, 2048), (1, 64, 300, 77), (2, 32, 1024, 256),
                                   (1, 256, 2048, 1024), (2, 128, 700, 77), (1, 128, 40, 33), (2, 128, 9, 9),
                                   (1, 128, 5000, 1000)])
def test_decode_over_the_fp8_cache(capi, dev, shape):
    B, H, N, topk = shape
    gen = torch.Generator().manual_seed(sum(shape))
    q, kv, idx = mla.mla_make_inputs(B, H, N, topk, generator=gen)
    idx[0, 3] = -1                            # padding, out-of-range and repeated entries
    idx[0, 5] = N
    idx[-1, 7] = idx[-1, 8]
    cache = make_cache(capi, dev, kv)
    got32 = run_fp8(capi, dev, q, cache, idx, torch.float32)
    ref = mla.sparse_mla_decode_fp8(q, cache, idx, out_dtype=torch.float32)
    assert mla.rel_rms_error(got32, ref) <= TOL
    # the same kernel on the dequantised cache: bit for bit, both output types
    deq = mla.latent_dequantize(cache.cpu())
    assert torch.equal(got32, run_bf16(capi, dev, q, deq, idx, torch.float32))
    assert torch.equal(run_fp8(capi, dev, q, cache, idx), run_bf16(capi, dev, q, deq, idx))
    # config 5000+n asks for the two-step form (dequantise into the workspace, then the bf16 kernels): same bits
    assert torch.equal(run_fp8(capi, dev, q, cache, idx, torch.float32, config=5000), got32)
    # and not far from the attention over the unquantised rows (e4m3 keeps 3 mantissa bits)
    exact = mla.sparse_mla_decode(q, kv, idx, out_dtype=torch.float32)
    assert ((got32 - exact).pow(2).mean().sqrt() / exact.pow(2).mean().sqrt()).item() <= 0.1


def test_all_padding_and_forced_splits(capi, dev):
    gen = torch.Generator().manual_seed(5)
    q, kv, idx = mla.mla_make_inputs(2, 128, 1024, 256, generator=gen)
    cache = make_cache(capi, dev, kv)
    idx[1] = -1                               # a request without any selected row: zeros
    out = run_fp8(capi, dev, q, cache, idx, torch.float32, config=3)
    assert (out[1] == 0).all()
    assert torch.equal(run_fp8(capi, dev, q, cache, idx, torch.float32, config=5003), out)
    ref = mla.sparse_mla_decode_fp8(q[:1], cache[:1], idx[:1], out_dtype=torch.float32)
    assert mla.rel_rms_error(out[:1], ref) <= TOL


def test_full_workload_shape(capi, dev):
    B, H, N, topk = 64, 128, 32768, 2048
    gen = torch.Generator(device=dev).manual_seed(20264)
    q = torch.randn(B, H, 576, device=dev, generator=gen).bfloat16()
    cache = torch.empty(B, N, 656, dtype=torch.uint8, device=dev)
    for b0 in range(0, B, 8):                 # the bf16 rows of 8 requests at a time (302 MB)
        kv = torch.randn(8, N, 576, device=dev, generator=gen).bfloat16()
        capi.mla_latent_quant_launch(cache[b0:b0 + 8], kv)
    idx = torch.stack([torch.randperm(N, device=dev, generator=gen)[:topk] for _ in range(B)]).int()
    out = torch.empty(B, H, 512, device=dev)
    ws = torch.empty(capi.sparse_mla_fp8_workspace_bytes(B, H, topk), dtype=torch.uint8, device=dev)
    capi.sparse_mla_decode_fp8_launch(out, q, cache, idx, ws)
    torch.cuda.synchronize()
    for b0 in range(0, B, 16):
        deq = mla.latent_dequantize_device(cache[b0:b0 + 16])
        ref = mla.sparse_mla_decode(q[b0:b0 + 16], deq, idx[b0:b0 + 16], out_dtype=torch.float32)
        assert mla.rel_rms_error(out[b0:b0 + 16], ref) <= TOL


def test_rejects_bad_arguments(capi, dev):
    q = torch.zeros(1, 128, 576, dtype=torch.bfloat16, device=dev)
    cache = torch.zeros(1, 64, 656, dtype=torch.uint8, device=dev)
    idx = torch.zeros(1, 32, dtype=torch.int32, device=dev)
    out = torch.empty(1, 128, 512, dtype=torch.bfloat16, device=dev)
    with pytest.raises(capi.LaunchRejected):  # workspace of the bf16 launcher: too small for the compact block
        capi.sparse_mla_decode_fp8_launch(out, q, cache, idx,
                                          torch.empty(capi.sparse_mla_workspace_bytes(1, 128, 32), dtype=torch.uint8, device=dev))
    torch.cuda.synchronize()


@pytest.mark.parametrize('page', [16, 64])
def test_paged_fp8_cache(capi, dev, page):
    # the pages of a contiguous e4m3 cache scattered into a pool: the same result bit for bit, with a block table
    # (logical positions) and without one (pool rows); an unmapped page is padding
    gen = torch.Generator().manual_seed(60 + page)
    B, H, N, topk = 3, 128, 1024, 256
    q, kv, idx = mla.mla_make_inputs(B, H, N, topk, generator=gen)
    cache = make_cache(capi, dev, kv)
    per_req = N // page
    n_pages = B * per_req + 3
    order = torch.randperm(n_pages, generator=gen)[:B * per_req]
    pool = torch.randint(0, 255, (n_pages, page, 656), generator=gen).to(torch.uint8)
    pool[order] = cache.cpu().reshape(B * per_req, page, 656)
    table = order.reshape(B, per_req).int()
    want = run_fp8(capi, dev, q, cache, idx, torch.float32)

    def run_paged(table_arg, idx_arg):
        out = torch.full((B, H, 512), float('nan'), device=dev)
        ws = torch.empty(capi.sparse_mla_fp8_workspace_bytes(B, H, topk), dtype=torch.uint8, device=dev)
        capi.sparse_mla_decode_fp8_paged_launch(out, q.to(dev), pool.to(dev), None if table_arg is None else table_arg.to(dev),
                                                idx_arg.to(dev), ws)
        torch.cuda.synchronize()
        return out.cpu()

    assert torch.equal(run_paged(table, idx), want)
    rows = mla.resolve_paged_indices(idx, table, page, n_pages * page).int()
    assert torch.equal(run_paged(None, rows), want)
    # one page of request 1 unmapped: its positions become padding
    table2 = table.clone()
    table2[1, 2] = -1
    idx_masked = idx.clone()
    idx_masked[1][(idx[1] >= 2 * page) & (idx[1] < 3 * page)] = -1
    assert torch.equal(run_paged(table2, idx), run_fp8(capi, dev, q, cache, idx_masked, torch.float32))
