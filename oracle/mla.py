"""Oracle for sparse-MLA decode attention (test infrastructure only).

Specification restated (workload config 3): per request b, all heads attend to the rows of the
request's latent cache selected by ``idx[b]``::

    K_g = kv[b, idx[b]]                      [topk, 576]
    s   = q[b] @ K_g.T * sm_scale            [heads, topk]     sm_scale = 192**-0.5
    out = softmax(s) @ K_g[:, :512]          [heads, 512] -> bf16

bf16 inputs are upcast and all arithmetic is fp32. Index values < 0 or >= N are padding and
take no part in the softmax. The reference repository has no implementation of this operator;
only its model contract (agent_workdir/model.py:9-26) shapes the functions below.

Pinned by (tests/test_oracle_mla.py):
  * ``sparse_mla_loops_f64``: float64 scalar loops written straight from the definition;
  * library special case: idx = arange(N) equals ``scaled_dot_product_attention`` with one
    shared KV head;
  * invariants: permutation of idx, all-equal V rows, shift invariance, split-and-merge by
    log-sum-exp.

Paged cache (the serving-side layout next to the operator; no counterpart in the reference
repository either): ``resolve_paged_indices`` maps logical positions through a block table,
position p of request b -> row ``p % page_size`` of page ``block_table[b, p // page_size]`` of
one pool shared by all requests. Pinned by scalar loops over divmod on small cases and by the
identity "scatter a contiguous cache's pages into a pool under a random page permutation ->
the paged result equals the contiguous result exactly".

``index_scores`` is the scoring in front of the selection (the indexer of DeepSeek sparse attention on one
decode step: per-head ReLU of scaled q.k, weighted sum over the index heads). Pinned by scalar loops in
float64, by its invariants (non-negative weights give non-negative scores, a head with weight 0 drops out,
scores are linear in w) and by a golden fixture from the third-party ``transformers`` indexer module, whose
returned top-k indices must equal the top-k of these scores (tests/golden/make_indexer_golden.py).

``topk_select`` is the selection that produces ``idx`` from index scores. Pinned by ``torch.topk`` as
a set on tie-free rows, by scalar loops with an explicit (value, index) ordering on rows full of
ties, signed zeros, infinities and NaNs, and by its invariants (ascending indices, every chosen
score >= every unchosen one).
"""

import math

import numpy as np
import torch

D_QK = 576
D_V = 512
SM_SCALE = 192 ** -0.5


def sparse_mla_decode(q, kv, idx, sm_scale=SM_SCALE, out_dtype=torch.bfloat16):
    """q [B,H,576], kv [B,N,576], idx [B,topk] int32 -> out [B,H,512] (fp32 math)."""
    B, H, _ = q.shape
    N = kv.shape[1]
    valid = (idx >= 0) & (idx < N)
    safe = idx.clamp(0, N - 1).long()
    kg = torch.gather(kv, 1, safe[:, :, None].expand(-1, -1, kv.shape[2])).float()
    s = torch.einsum('bhd,bkd->bhk', q.float(), kg) * sm_scale
    s = s.masked_fill(~valid[:, None, :], float('-inf'))
    p = torch.softmax(s, dim=-1)
    out = torch.einsum('bhk,bkd->bhd', p, kg[:, :, :D_V])
    return out.to(out_dtype)


def sparse_mla_loops_f64(q, kv, idx, sm_scale=SM_SCALE):
    q = np.asarray(q, dtype=np.float64)
    kv = np.asarray(kv, dtype=np.float64)
    B, H, D = q.shape
    N = kv.shape[1]
    dv = min(D_V, D)
    out = np.zeros((B, H, dv))
    for b in range(B):
        rows = [int(i) for i in idx[b] if 0 <= int(i) < N]
        for h in range(H):
            scores = [sum(q[b, h, d] * kv[b, r, d] for d in range(D)) * sm_scale for r in rows]
            mx = max(scores)
            w = [math.exp(s - mx) for s in scores]
            tot = sum(w)
            for j in range(dv):
                out[b, h, j] = sum(wi * kv[b, r, j] for wi, r in zip(w, rows)) / tot
    return out


def mla_make_inputs(batch, n_heads, n_kv_rows, topk, generator=None, device='cpu'):
    """q, kv ~ N(0,1) cast to bf16; idx = the first topk entries of a per-request random
    permutation of the cache rows (unsorted, no repeats), int32."""
    gen = generator
    q = torch.randn(batch, n_heads, D_QK, generator=gen, device=device).bfloat16()
    kv = torch.randn(batch, n_kv_rows, D_QK, generator=gen, device=device).bfloat16()
    idx = torch.stack([torch.randperm(n_kv_rows, generator=gen, device=device)[:topk]
                       for _ in range(batch)]).int()
    return [q, kv, idx]


def resolve_paged_indices(idx, block_table, page_size, n_pool_rows):
    """Logical positions idx [B,topk] -> rows of the pool (int64), -1 for padding: negative
    positions, positions beyond the block table, unmapped (negative) pages, rows beyond the
    pool. With ``block_table=None`` idx already holds pool rows and only the range check
    applies."""
    idx = idx.long()
    if block_table is None:
        rows = idx
    else:
        max_pages = block_table.shape[1]
        page_no = torch.div(idx, page_size, rounding_mode='floor')
        inside = (idx >= 0) & (page_no < max_pages)
        page = torch.gather(block_table.long(), 1, page_no.clamp(0, max_pages - 1))
        rows = page * page_size + torch.remainder(idx, page_size)
        rows = torch.where(inside & (page >= 0), rows, torch.full_like(rows, -1))
    return torch.where((rows >= 0) & (rows < n_pool_rows), rows, torch.full_like(rows, -1))


def sparse_mla_decode_paged(q, kv_pool, block_table, idx, sm_scale=SM_SCALE, out_dtype=torch.bfloat16):
    """q [B,H,576], kv_pool [n_pages,page_size,576], block_table [B,max_pages] or None,
    idx [B,topk] -> out [B,H,512]: the attention of ``sparse_mla_decode`` over the rows the
    block table resolves to."""
    n_pages, page_size, d = kv_pool.shape
    rows = resolve_paged_indices(idx, block_table, page_size, n_pages * page_size)
    pool = kv_pool.reshape(1, n_pages * page_size, d).expand(q.shape[0], -1, -1)
    return sparse_mla_decode(q, pool, rows, sm_scale, out_dtype)


def mla_scatter_into_pool(kv, page_size, n_spare_pages=3, generator=None):
    """A contiguous cache kv [B,N,576] (N a multiple of page_size) cut into pages and placed in a
    pool at randomly permuted page numbers, with a few unused pages of noise in between.
    Returns (kv_pool [n_pages,page_size,576], block_table [B, N/page_size] int32)."""
    B, N, d = kv.shape
    assert N % page_size == 0
    per_req = N // page_size
    n_pages = B * per_req + n_spare_pages
    order = torch.randperm(n_pages, generator=generator)[:B * per_req]
    pool = torch.randn(n_pages, page_size, d, generator=generator).to(kv.dtype)
    pool[order] = kv.reshape(B * per_req, page_size, d).cpu()
    return pool, order.reshape(B, per_req).int()


def index_scores(q, k_cache, w, lengths=None, scale=128 ** -0.5):
    """Indexer scores of a decode step: q [B,Hi,d], k_cache [B,N,d] (bf16, taken to fp32), w [B,Hi] fp32 ->
    scores [B,N] fp32 = sum_h w[b,h] * relu(scale * q[b,h] . k_cache[b,t]); -inf at positions >= lengths[b]."""
    s = torch.einsum('bhd,bnd->bhn', q.float(), k_cache.float()) * scale
    out = torch.einsum('bh,bhn->bn', w.float(), torch.relu(s))
    if lengths is not None:
        pos = torch.arange(k_cache.shape[1], device=out.device)[None, :]
        out = out.masked_fill(pos >= lengths.to(out.device)[:, None].long(), float('-inf'))
    return out


LATENT_ROW_BYTES = 656      # 512 e4m3 codes + 4 fp32 scales + 64 bf16 rope values


def latent_quantize(kv, pow2=False):
    """The e4m3 storage form of latent cache rows: kv [..., 576] bf16 -> uint8 [..., 656]. Bytes [0,512): codes of
    the 512 latent values, quantised per block of 128 with scale = amax/448 (``pow2``: the smallest power of two that
    is at least that), exactly as the MoE activation quantiser (oracle.moe.quantize_groups); bytes [512,528): the 4
    scales, little-endian fp32; bytes [528,656): the 64 rope values as bf16, unchanged. The layout is the one
    third-party sparse-attention decoders document for an fp8 latent cache; no file of theirs is available here,
    so it is pinned by its own description only (parity unpinned against a third-party implementation)."""
    from oracle import moe
    lead = kv.shape[:-1]
    flat = kv.reshape(-1, 576)
    codes, scales = moe.quantize_groups(flat[:, :512].float(), pow2=pow2)
    out = torch.empty(flat.shape[0], LATENT_ROW_BYTES, dtype=torch.uint8)
    out[:, :512] = codes.view(torch.uint8)
    out[:, 512:528] = scales.contiguous().view(torch.uint8).reshape(-1, 16)
    out[:, 528:] = flat[:, 512:].contiguous().view(torch.uint8).reshape(-1, 128)
    return out.reshape(*lead, LATENT_ROW_BYTES)


def latent_dequantize(cache):
    """uint8 [..., 656] -> bf16 [..., 576]: code * scale in fp32, rounded to nearest-even bf16; rope as stored."""
    lead = cache.shape[:-1]
    flat = cache.reshape(-1, LATENT_ROW_BYTES)
    codes = e4m3_to_float(flat[:, :512])
    scales = flat[:, 512:528].contiguous().view(torch.float32)             # [rows, 4]
    latent = (codes.reshape(-1, 4, 128) * scales[:, :, None]).reshape(-1, 512).bfloat16()
    rope = flat[:, 528:].contiguous().view(torch.bfloat16)
    return torch.cat([latent, rope], dim=1).reshape(*lead, 576)


def latent_dequantize_device(cache):
    """latent_dequantize on whatever device the cache is on (the codes through torch's own e4m3 cast)."""
    lead = cache.shape[:-1]
    flat = cache.reshape(-1, LATENT_ROW_BYTES)
    codes = flat[:, :512].contiguous().view(torch.float8_e4m3fn).float()
    scales = flat[:, 512:528].contiguous().view(torch.float32)
    latent = (codes.reshape(-1, 4, 128) * scales[:, :, None]).reshape(-1, 512).bfloat16()
    rope = flat[:, 528:].contiguous().view(torch.bfloat16)
    return torch.cat([latent, rope], dim=1).reshape(*lead, 576)


def sparse_mla_decode_fp8(q, cache, idx, **kwargs):
    """sparse_mla_decode over a cache in the 656-byte form: attention over the dequantised rows."""
    return sparse_mla_decode(q, latent_dequantize(cache.cpu()), idx, **kwargs)


def e4m3_to_float(codes):
    """OCP e4m3 codes (uint8 tensor) -> fp32, from the bit fields: sign 1, exponent 4 (bias 7), mantissa 3;
    exponent 0 is subnormal (mantissa / 8 * 2^-6), code 0x7f / 0xff is NaN, there are no infinities."""
    c = codes.to(torch.int32)
    sign = torch.where((c >> 7) == 1, -1.0, 1.0)
    exp = (c >> 3) & 15
    man = (c & 7).float()
    normal = (1.0 + man / 8.0) * torch.pow(2.0, (exp - 7).float())
    subnormal = man / 8.0 * 2.0 ** -6
    val = torch.where(exp == 0, subnormal, normal)
    val = torch.where((c & 0x7f) == 0x7f, torch.full_like(val, float('nan')), val)
    return (sign * val).float()


def index_scores_fp8(q_codes, k_codes, k_scale, w, lengths=None, scale=128 ** -0.5):
    """Indexer scores over e4m3 keys: q_codes [B,Hi,d] and k_codes [B,N,d] uint8 e4m3 codes, k_scale [B,N]
    fp32 (key = code * k_scale), w [B,Hi] fp32 (head weight times the scale of that head's q) ->
    scores [B,N] fp32 = k_scale[b,t] * sum_h w[b,h] * relu(scale * q[b,h] . k[b,t]); -inf at positions >=
    lengths[b]. The quantised form of ``index_scores`` (the third-party model file
    transformers/models/deepseek_v32/modeling_deepseek_v32.py:203-212 states that its bf16 scoring stands
    for an `fp8_index` kernel of the same formula); evaluated in float64."""
    q = e4m3_to_float(q_codes).double()
    k = e4m3_to_float(k_codes).double()
    s = torch.relu(torch.einsum('bhd,bnd->bhn', q, k) * scale)
    out = (torch.einsum('bh,bhn->bn', w.double(), s) * k_scale.double()).float()
    if lengths is not None:
        pos = torch.arange(k_codes.shape[1], device=out.device)[None, :]
        out = out.masked_fill(pos >= lengths.to(out.device)[:, None].long(), float('-inf'))
    return out


def topk_select(scores, k, lengths=None):
    """Indices of the k largest scores per row among the first lengths[b] entries (all, if None):
    ties to the lower index, ascending index order, -1 where fewer than k candidates exist; NaN ranks
    below every number (-inf included). int32 [B, k]."""
    B, n = scores.shape
    out = torch.full((B, k), -1, dtype=torch.int32)
    for b in range(B):
        valid = n if lengths is None else max(0, min(n, int(lengths[b])))
        row = scores[b, :valid].double()
        nan = torch.isnan(row)
        # stable descending sort of (is-number, value): numbers first, equal values by index
        row = torch.where(nan, torch.full_like(row, float('-inf')), row)
        order = torch.sort(row, descending=True, stable=True).indices
        numbers = order[~nan[order]]
        nans = order[nan[order]]
        chosen = torch.cat([numbers, nans])[:k]
        out[b, :chosen.numel()] = torch.sort(chosen).values.int()
    return out


def rel_rms_error(actual, expected):
    """max |a - e| / rms(e): the figure the 2e-2 bound of this operator is stated on."""
    a = actual.double()
    e = expected.double()
    return ((a - e).abs().max() / e.pow(2).mean().sqrt()).item()
