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
