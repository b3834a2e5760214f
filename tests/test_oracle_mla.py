"""Pins the sparse-MLA oracle: brute force, the dense library special case and invariants."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import mla


def _inputs(seed=0, B=2, H=4, N=40, topk=12):
    gen = torch.Generator().manual_seed(seed)
    return mla.mla_make_inputs(B, H, N, topk, generator=gen)


def test_matches_float64_loops():
    q, kv, idx = _inputs()
    want = mla.sparse_mla_loops_f64(q.float().numpy(), kv.float().numpy(), idx.numpy())
    got = mla.sparse_mla_decode(q, kv, idx, out_dtype=torch.float32)
    np.testing.assert_allclose(got.numpy(), want, rtol=2e-5, atol=2e-6)


def test_dense_special_case_is_library_attention():
    q, kv, _ = _inputs(1, B=2, H=8, N=64)
    idx = torch.arange(64, dtype=torch.int32).expand(2, 64).contiguous()
    got = mla.sparse_mla_decode(q, kv, idx, out_dtype=torch.float32)
    k = kv.float()[:, None]                       # one KV head shared by every query head
    want = F.scaled_dot_product_attention(q.float()[:, :, None, :], k.expand(-1, 8, -1, -1),
                                          k[..., :512].expand(-1, 8, -1, -1), scale=mla.SM_SCALE)
    torch.testing.assert_close(got, want[:, :, 0], rtol=1e-5, atol=1e-6)


def test_index_order_does_not_matter():
    q, kv, idx = _inputs(2)
    perm = torch.randperm(idx.shape[1], generator=torch.Generator().manual_seed(3))
    a = mla.sparse_mla_decode(q, kv, idx, out_dtype=torch.float32)
    b = mla.sparse_mla_decode(q, kv, idx[:, perm], out_dtype=torch.float32)
    torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-6)


def test_only_selected_rows_matter():
    q, kv, idx = _inputs(4)
    kv2 = kv.clone()
    mask = torch.ones(kv.shape[:2], dtype=torch.bool)
    mask.scatter_(1, idx.long(), False)
    kv2[mask] = 7.0
    assert torch.equal(mla.sparse_mla_decode(q, kv, idx), mla.sparse_mla_decode(q, kv2, idx))


def test_equal_value_rows_give_that_row():
    q, kv, idx = _inputs(5)
    kv[:, :, :512] = kv[:, :1, :512]
    out = mla.sparse_mla_decode(q, kv, idx, out_dtype=torch.float32)
    torch.testing.assert_close(out, kv[:, :1, :512].float().expand_as(out), rtol=1e-5, atol=1e-6)


def test_padding_entries_are_ignored():
    q, kv, idx = _inputs(6)
    padded = torch.cat([idx[:, :5], torch.full((2, 3), -1, dtype=torch.int32), idx[:, 5:],
                        torch.full((2, 2), 40, dtype=torch.int32)], dim=1)
    assert torch.equal(mla.sparse_mla_decode(q, kv, idx), mla.sparse_mla_decode(q, kv, padded))


def test_split_and_merge_by_log_sum_exp():
    q, kv, idx = _inputs(7, topk=24)
    full = mla.sparse_mla_decode(q, kv, idx, out_dtype=torch.float32)
    parts, lses = [], []
    for piece in idx.split(8, dim=1):
        kg = torch.gather(kv, 1, piece.long()[:, :, None].expand(-1, -1, 576)).float()
        s = torch.einsum('bhd,bkd->bhk', q.float(), kg) * mla.SM_SCALE
        lses.append(torch.logsumexp(s, -1))
        parts.append(mla.sparse_mla_decode(q, kv, piece, out_dtype=torch.float32))
    w = torch.softmax(torch.stack(lses, 0), 0)
    merged = (torch.stack(parts, 0) * w[..., None]).sum(0)
    torch.testing.assert_close(merged, full, rtol=1e-5, atol=1e-6)


def test_output_dtype_and_shape():
    q, kv, idx = _inputs(8)
    out = mla.sparse_mla_decode(q, kv, idx)
    assert out.dtype == torch.bfloat16 and out.shape == (2, 4, 512)
    assert idx.dtype == torch.int32
    for b in range(2):
        assert len(set(idx[b].tolist())) == idx.shape[1]


# ---- paged cache ------------------------------------------------------------------------------

def _resolve_by_loops(idx, block_table, page_size, n_pool_rows):
    out = []
    for b, row in enumerate(idx.tolist()):
        res = []
        for p in row:
            r = -1
            if block_table is None:
                r = p
            elif p >= 0:
                page_no, offset = divmod(p, page_size)
                if page_no < block_table.shape[1] and int(block_table[b, page_no]) >= 0:
                    r = int(block_table[b, page_no]) * page_size + offset
            res.append(r if 0 <= r < n_pool_rows else -1)
        out.append(res)
    return torch.tensor(out)


def test_paged_resolution_matches_divmod_loops():
    gen = torch.Generator().manual_seed(5)
    page_size, n_pages, B, max_pages = 4, 9, 3, 5
    table = torch.randint(-1, n_pages + 2, (B, max_pages), generator=gen).int()   # unmapped and out-of-pool pages
    idx = torch.randint(-3, max_pages * page_size + 6, (B, 40), generator=gen).int()
    got = mla.resolve_paged_indices(idx, table, page_size, n_pages * page_size)
    assert torch.equal(got, _resolve_by_loops(idx, table, page_size, n_pages * page_size))
    assert (got == -1).any() and (got >= 0).any()
    rows = torch.randint(-2, n_pages * page_size + 3, (B, 40), generator=gen).int()
    got = mla.resolve_paged_indices(rows, None, page_size, n_pages * page_size)
    assert torch.equal(got, _resolve_by_loops(rows, None, page_size, n_pages * page_size))


def test_paged_equals_contiguous_when_the_pool_holds_the_same_pages():
    gen = torch.Generator().manual_seed(6)
    q, kv, idx = mla.mla_make_inputs(3, 4, 48, 20, generator=gen)
    idx[1, 3] = -1
    idx[2, 7] = 48
    want = mla.sparse_mla_decode(q, kv, idx, out_dtype=torch.float32)
    pool, table = mla.mla_scatter_into_pool(kv, 8, generator=gen)
    got = mla.sparse_mla_decode_paged(q, pool, table, idx, out_dtype=torch.float32)
    assert torch.equal(got, want)
    # the same selection handed over as pool rows, without a block table
    rows = mla.resolve_paged_indices(idx, table, 8, pool.shape[0] * 8).int()
    assert torch.equal(mla.sparse_mla_decode_paged(q, pool, None, rows, out_dtype=torch.float32), want)


def test_unmapped_pages_drop_their_positions():
    gen = torch.Generator().manual_seed(7)
    q, kv, idx = mla.mla_make_inputs(2, 4, 32, 16, generator=gen)
    pool, table = mla.mla_scatter_into_pool(kv, 8, generator=gen)
    table[0, 1] = -1
    keep = idx.clone()
    keep[0][(idx[0] >= 8) & (idx[0] < 16)] = -1
    want = mla.sparse_mla_decode(q, kv, keep, out_dtype=torch.float32)
    assert torch.equal(mla.sparse_mla_decode_paged(q, pool, table, idx, out_dtype=torch.float32), want)


# ---- top-k selection of index scores -----------------------------------------------------------

def _select_by_loops(scores, k, lengths):
    out = []
    for b, row in enumerate(scores.tolist()):
        valid = len(row) if lengths is None else max(0, min(len(row), int(lengths[b])))
        # rank: numbers before NaN, larger first (-0 == +0), then lower index
        ranked = sorted(range(valid), key=lambda i: (row[i] != row[i], 0.0 if row[i] != row[i] else -row[i], i))
        chosen = sorted(ranked[:k])
        out.append(chosen + [-1] * (k - len(chosen)))
    return torch.tensor(out, dtype=torch.int32)


def test_topk_select_is_torch_topk_on_tie_free_rows():
    gen = torch.Generator().manual_seed(31)
    scores = torch.randn(5, 300, generator=gen)
    got = mla.topk_select(scores, 40)
    want = torch.topk(scores, 40, dim=1).indices.sort(dim=1).values.int()
    assert torch.equal(got, want)


def test_topk_select_ties_specials_and_lengths():
    gen = torch.Generator().manual_seed(32)
    scores = torch.randint(-3, 4, (6, 50), generator=gen).float()       # many ties
    scores[0, 5] = float('inf')
    scores[1, 7] = float('-inf')
    scores[2, 3::7] = float('nan')
    scores[3, ::2] = -0.0
    scores[3, 1::2] = 0.0
    lengths = torch.tensor([50, 50, 50, 50, 9, 0], dtype=torch.int32)
    for k in (1, 8, 20, 50, 64):
        for ln in (None, lengths):
            got = mla.topk_select(scores, k, ln)
            assert torch.equal(got, _select_by_loops(scores, k, ln)), (k, ln)
    # invariants on the last call: ascending, -1 padding at the end, chosen >= unchosen
    got = mla.topk_select(scores, 8)
    for b in range(6):
        row = got[b]
        assert (row[1:] > row[:-1]).all()
        if not torch.isnan(scores[b]).any():
            unchosen = torch.ones(50, dtype=torch.bool)
            unchosen[row.long()] = False
            assert scores[b, row.long()].min() >= scores[b, unchosen].max()


# ---- indexer scores ------------------------------------------------------------------------------

def test_index_scores_match_float64_loops_and_invariants():
    gen = torch.Generator().manual_seed(33)
    B, Hi, N, d = 2, 4, 9, 16
    q = torch.randn(B, Hi, d, generator=gen).bfloat16()
    k = torch.randn(B, N, d, generator=gen).bfloat16()
    w = torch.randn(B, Hi, generator=gen)
    lengths = torch.tensor([9, 5], dtype=torch.int32)
    got = mla.index_scores(q, k, w, lengths, scale=0.25)
    for b in range(B):
        for t in range(N):
            if t >= int(lengths[b]):
                assert got[b, t] == float('-inf')
                continue
            want = sum(float(w[b, h]) * max(0.0, 0.25 * sum(float(q[b, h, j]) * float(k[b, t, j]) for j in range(d)))
                       for h in range(Hi))
            assert abs(float(got[b, t]) - want) <= 1e-5 * (1 + abs(want))
    assert (mla.index_scores(q, k, w.abs()) >= 0).all()
    w0 = w.clone()
    w0[:, 1] = 0
    q_other = q.clone()
    q_other[:, 1] = 7.0
    assert torch.equal(mla.index_scores(q, k, w0), mla.index_scores(q_other, k, w0))       # a head of weight 0 drops out
    torch.testing.assert_close(mla.index_scores(q, k, 3 * w), 3 * mla.index_scores(q, k, w), rtol=1e-6, atol=1e-6)


def test_index_scores_fp8_decode_loops_and_agreement_with_the_bf16_form():
    from oracle import moe
    # the decoder against an independent one (torch's cast), all 256 codes
    codes = torch.arange(256, dtype=torch.uint8)
    mine, theirs = mla.e4m3_to_float(codes), codes.view(torch.float8_e4m3fn).float()
    assert torch.equal(torch.isnan(mine), torch.isnan(theirs))
    assert torch.equal(mine[~torch.isnan(mine)], theirs[~torch.isnan(theirs)])
    # plain float64 loops on a tiny case
    gen = torch.Generator().manual_seed(35)
    B, Hi, N, d = 2, 3, 7, 8
    qc = torch.randint(0, 0x7f, (B, Hi, d), generator=gen).to(torch.uint8) | (torch.randint(0, 2, (B, Hi, d), generator=gen) << 7).to(torch.uint8)
    kc = torch.randint(0, 0x7f, (B, N, d), generator=gen).to(torch.uint8) | (torch.randint(0, 2, (B, N, d), generator=gen) << 7).to(torch.uint8)
    ks = torch.rand(B, N, generator=gen) + 0.5
    w = torch.randn(B, Hi, generator=gen)
    lengths = torch.tensor([7, 4], dtype=torch.int32)
    got = mla.index_scores_fp8(qc, kc, ks, w, lengths, scale=2.0 ** -10)
    qf, kf = qc.view(torch.float8_e4m3fn).double(), kc.view(torch.float8_e4m3fn).double()
    for b in range(B):
        for t in range(N):
            if t >= int(lengths[b]):
                assert got[b, t] == float('-inf')
                continue
            want = float(ks[b, t]) * sum(float(w[b, h]) * max(0.0, 2.0 ** -10 * sum(float(qf[b, h, j]) * float(kf[b, t, j]) for j in range(d)))
                                         for h in range(Hi))
            assert abs(float(got[b, t]) - want) <= 1e-6 * (1 + abs(want))
    # the quantised form of the bf16 scores: on keys and queries that e4m3 holds exactly (scales a power of two)
    # both oracles agree, and on quantised random inputs the scores stay within the quantisation error
    B, Hi, N, d = 2, 8, 64, 128
    q = torch.randn(B, Hi, d, generator=gen)
    k = torch.randn(B, N, d, generator=gen)
    w = torch.randn(B, Hi, generator=gen) * Hi ** -0.5
    qq, qs = moe.quantize_groups(q.reshape(B * Hi, d), pow2=True)
    kq, ks = moe.quantize_groups(k.reshape(B * N, d), pow2=True)
    q_deq = (qq.float() * qs).reshape(B, Hi, d)
    k_deq = (kq.float() * ks).reshape(B, N, d)
    assert torch.equal(q_deq.bfloat16().float(), q_deq) and torch.equal(k_deq.bfloat16().float(), k_deq)
    fp8 = mla.index_scores_fp8(qq.view(torch.uint8).reshape(B, Hi, d), kq.view(torch.uint8).reshape(B, N, d),
                               ks.reshape(B, N), w * qs.reshape(B, Hi))
    torch.testing.assert_close(fp8, mla.index_scores(q_deq.bfloat16(), k_deq.bfloat16(), w), rtol=1e-5, atol=1e-5)
    exact = mla.index_scores(q.bfloat16(), k.bfloat16(), w)
    assert mla.rel_rms_error(fp8, exact) < 0.5      # (e4m3 keeps 3 mantissa bits: the scores move by a few per cent)
    assert torch.nn.functional.cosine_similarity(fp8.flatten(), exact.flatten(), dim=0) > 0.99


def test_index_scores_select_what_the_third_party_indexer_selects():
    from pathlib import Path
    z = np.load(Path(__file__).parent / 'golden' / 'indexer_golden.npz')
    q, k, w = (torch.from_numpy(z[n]) for n in ('q', 'k', 'w'))
    scores = mla.index_scores(q, k, w, scale=float(z['scale'][0]))
    idx = mla.topk_select(scores, z['topk'].shape[1])
    np.testing.assert_array_equal(idx.numpy(), z['topk'])


# ---- e4m3 storage form of the latent cache ---------------------------------------------------------------

def test_latent_cache_layout_round_trip_and_error_bound():
    import struct
    gen = torch.Generator().manual_seed(41)
    kv = (torch.randn(5, 576, generator=gen) * 3).bfloat16()
    kv[1, 128:256] = 0
    for pow2 in (False, True):
        cache = mla.latent_quantize(kv, pow2=pow2)
        assert cache.shape == (5, mla.LATENT_ROW_BYTES) and cache.dtype == torch.uint8
        # the layout, field by field, with plain loops
        for r in range(5):
            row = bytes(cache[r].tolist())
            scales = struct.unpack('<4f', row[512:528])
            for blk in range(4):
                vals = kv[r, 128 * blk:128 * blk + 128].float()
                amax = max(float(vals.abs().max()), 1e-12)
                if pow2:
                    assert scales[blk] >= amax / 448 * (1 - 1e-6) and scales[blk] / 2 < amax / 448
                    m, _ = np.frexp(scales[blk])
                    assert m == 0.5
                else:
                    assert abs(scales[blk] - amax / 448) <= 1e-6 * amax / 448
                for j in (0, 17, 127):
                    code = torch.tensor([row[128 * blk + j]], dtype=torch.uint8).view(torch.float8_e4m3fn).float().item()
                    want = float(vals[j]) / scales[blk]
                    assert abs(code - want) <= max(abs(want) * 2.0 ** -4, 2.0 ** -10)
            rope = torch.tensor(list(row[528:]), dtype=torch.uint8).view(torch.bfloat16)
            assert torch.equal(rope, kv[r, 512:])
        deq = mla.latent_dequantize(cache)
        assert torch.equal(deq, mla.latent_dequantize_device(cache))
        assert torch.equal(deq[:, 512:], kv[:, 512:])
        blocks = kv[:, :512].float().reshape(5, 4, 128)
        bound = blocks.abs().amax(dim=-1, keepdim=True) * (2.0 ** -4 + 2.0 ** -8) * (2 if pow2 else 1)
        assert ((deq[:, :512].float().reshape(5, 4, 128) - blocks).abs() <= bound + 1e-30).all()
    # values e4m3 holds exactly with a power-of-two block maximum survive the round trip unchanged
    exact = torch.zeros(2, 576)
    exact[:, :512] = torch.randint(-8, 9, (2, 512), generator=gen).float() * 0.25
    exact[:, 0:512:128] = 448 * 2.0 ** -6
    exact = exact.bfloat16()
    assert torch.equal(mla.latent_dequantize(mla.latent_quantize(exact, pow2=True)), exact)
    # attention over the fp8 cache = attention over the dequantised rows
    q, kv2, idx = mla.mla_make_inputs(2, 4, 64, 16, generator=gen)
    cache = mla.latent_quantize(kv2)
    assert torch.equal(mla.sparse_mla_decode_fp8(q, cache, idx), mla.sparse_mla_decode(q, mla.latent_dequantize(cache), idx))
