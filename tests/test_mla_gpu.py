"""GPU parity of sparse-MLA decode against the oracle, through the C ABI.

Tolerance: max |out - ref| <= 2e-2 * rms(ref), ref = fp32 oracle on the same bf16 inputs, checked
on the launcher's fp32 output (the values before the final rounding). The bf16 output is then
required to be exactly the round-to-nearest of those values; rounding to bf16 alone moves an
element by up to 2^-9 of its magnitude, which for the heavy-tailed outputs of this operator
(max|x| up to 9 rms at top-k 2048) already exceeds 2e-2 rms, so the bf16 output is held to
2e-2 rms plus that floor, measured on the reference itself.
The gather is exact (indices are used verbatim), which the 'equal value rows' and 'only selected
rows are read' cases check bit for bit."""
import os
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from oracle import mla

pytestmark = pytest.mark.gpu
TOL = 2e-2


def run_kernel(capi, q, kv, idx, config=0, dtype=torch.bfloat16):
    B, H, _ = q.shape
    out = torch.full((B, H, 512), float('nan'), device=q.device, dtype=dtype)
    ws = torch.empty(capi.sparse_mla_workspace_bytes(B, H, idx.shape[1], config), dtype=torch.uint8,
                     device=q.device)
    capi.sparse_mla_decode_launch(out, q, kv, idx, ws, config=config)
    torch.cuda.synchronize()
    return out


def oracle_on_gpu(q, kv, idx):
    return mla.sparse_mla_decode(q, kv, idx, out_dtype=torch.float32)


def check(capi, q, kv, idx, config, ref):
    exact = run_kernel(capi, q, kv, idx, config, torch.float32)
    out = run_kernel(capi, q, kv, idx, config)
    assert torch.isfinite(exact).all()
    err = mla.rel_rms_error(exact, ref)
    assert err <= TOL, err
    assert torch.equal(out, exact.bfloat16())     # the bf16 output is the rounded fp32 output
    floor = mla.rel_rms_error(ref.bfloat16().float(), ref)
    assert mla.rel_rms_error(out.float(), ref) <= TOL + floor
    return out


@pytest.mark.parametrize('config', [0, 1, 2, 5])
@pytest.mark.parametrize('shape', [(2, 128, 300, 96), (3, 32, 100, 33), (1, 64, 512, 257),
                                   (2, 128, 4096, 2048), (1, 256, 200, 64), (5, 128, 64, 1),
                                   # batches that are multiples of 8: the splits of a request share an XCD
                                   (8, 128, 600, 200), (16, 256, 300, 130), (8, 128, 2048, 1024), (24, 128, 90, 70)])
def test_matches_oracle(capi, dev, shape, config):
    B, H, N, topk = shape
    gen = torch.Generator().manual_seed(B * 1000 + topk)
    q, kv, idx = (t.to(dev) for t in mla.mla_make_inputs(B, H, N, topk, generator=gen))
    check(capi, q, kv, idx, config, oracle_on_gpu(q, kv, idx))


def test_against_cpu_oracle_small(capi, dev):
    gen = torch.Generator().manual_seed(77)
    q, kv, idx = mla.mla_make_inputs(2, 128, 500, 200, generator=gen)
    ref = mla.sparse_mla_decode(q, kv, idx, out_dtype=torch.float32)
    out = check(capi, q.to(dev), kv.to(dev), idx.to(dev), 0, ref.to(dev))
    # the reference harness's own bound, against the oracle's bf16 output
    torch.testing.assert_close(out.cpu(), ref.bfloat16(), atol=1e-2, rtol=1e-2)


def test_padding_and_out_of_range_entries(capi, dev):
    gen = torch.Generator().manual_seed(9)
    q, kv, idx = (t.to(dev) for t in mla.mla_make_inputs(2, 128, 700, 150, generator=gen))
    padded = torch.cat([idx[:, :40], torch.full((2, 30), -1, dtype=torch.int32, device=dev),
                        idx[:, 40:], torch.full((2, 11), 700, dtype=torch.int32, device=dev),
                        torch.full((2, 64), -1, dtype=torch.int32, device=dev)], dim=1).contiguous()
    ref = oracle_on_gpu(q, kv, padded)
    check(capi, q, kv, idx, 1, ref)
    check(capi, q, kv, padded, 1, ref)
    # a split made only of padding (the trailing 64 entries with 8 splits) contributes nothing
    check(capi, q, kv, padded, 8, ref)


def test_equal_value_rows_give_that_row_exactly(capi, dev):
    gen = torch.Generator().manual_seed(10)
    q, kv, idx = (t.to(dev) for t in mla.mla_make_inputs(2, 128, 300, 128, generator=gen))
    kv[:, :, :512] = kv[:, :1, :512]
    out = run_kernel(capi, q, kv, idx)
    want = kv[:, :1, :512].float().expand(2, 128, 512)
    # every probability-weighted sum of identical bf16 rows is that row up to the bf16
    # rounding of the probabilities (relative 2^-8) and of the output
    torch.testing.assert_close(out.float(), want, rtol=2 ** -6, atol=1e-3)


def test_only_selected_rows_are_read(capi, dev):
    gen = torch.Generator().manual_seed(11)
    q, kv, idx = (t.to(dev) for t in mla.mla_make_inputs(2, 128, 400, 100, generator=gen))
    a = run_kernel(capi, q, kv, idx, config=2)
    mask = torch.ones(kv.shape[:2], dtype=torch.bool, device=dev)
    mask.scatter_(1, idx.long(), False)
    kv2 = kv.clone()
    kv2[mask] = float('nan')
    b = run_kernel(capi, q, kv2, idx, config=2)
    assert torch.equal(a, b)                      # bit-exact: unselected rows never enter


def test_split_counts_agree(capi, dev):
    gen = torch.Generator().manual_seed(12)
    q, kv, idx = (t.to(dev) for t in mla.mla_make_inputs(2, 128, 2000, 1024, generator=gen))
    ref = oracle_on_gpu(q, kv, idx)
    outs = [run_kernel(capi, q, kv, idx, config=s, dtype=torch.float32) for s in (1, 2, 4, 8)]
    for o in outs:
        assert mla.rel_rms_error(o, ref) <= TOL
        assert mla.rel_rms_error(o, outs[0]) <= TOL


def test_one_wavefront_per_head_group_kernel_for_128_heads(capi, dev):
    # config 1000 + n selects the kernel that caches of 4 GB and more per request fall back to
    gen = torch.Generator().manual_seed(14)
    q, kv, idx = (t.to(dev) for t in mla.mla_make_inputs(2, 128, 900, 300, generator=gen))
    padded = torch.cat([idx[:, :100], torch.full((2, 20), -1, dtype=torch.int32, device=dev), idx[:, 100:]],
                       dim=1).contiguous()
    ref = oracle_on_gpu(q, kv, padded)
    for config in (1000, 1001, 1003):
        check(capi, q, kv, padded, config, ref)


def test_large_scores_do_not_overflow(capi, dev):
    gen = torch.Generator().manual_seed(13)
    q, kv, idx = (t.to(dev) for t in mla.mla_make_inputs(1, 128, 300, 200, generator=gen))
    q = (q.float() * 8).bfloat16()                # logits of a few hundred: one row dominates
    check(capi, q, kv, idx, 0, oracle_on_gpu(q, kv, idx))


def test_full_workload_shape(capi, dev):
    """Config 3 at full size: B=64, 128 heads, 32768-row caches (2.4 GB), top-k 2048."""
    B, H, N, topk = 64, 128, 32768, 2048
    gen = torch.Generator(device=dev).manual_seed(20253)
    q = torch.randn(B, H, 576, device=dev, generator=gen).bfloat16()
    kv = torch.randn(B, N, 576, device=dev, generator=gen).bfloat16()
    idx = torch.stack([torch.randperm(N, device=dev, generator=gen)[:topk] for _ in range(B)]).int()
    exact = run_kernel(capi, q, kv, idx, dtype=torch.float32)
    out = run_kernel(capi, q, kv, idx)
    assert torch.equal(out, exact.bfloat16())
    worst = 0.0
    for b0 in range(0, B, 8):                     # oracle in slices to bound its temporaries
        ref = oracle_on_gpu(q[b0:b0 + 8], kv[b0:b0 + 8], idx[b0:b0 + 8])
        worst = max(worst, mla.rel_rms_error(exact[b0:b0 + 8], ref))
    assert worst <= TOL, worst
    # index order is immaterial
    perm = torch.randperm(topk, device=dev, generator=gen)
    exact2 = run_kernel(capi, q, kv, idx[:, perm].contiguous(), dtype=torch.float32)
    assert mla.rel_rms_error(exact2, exact) <= TOL


def test_rejects_unsupported_shapes(capi, dev):
    q = torch.zeros(1, 48, 576, device=dev, dtype=torch.bfloat16)      # 48 heads: no kernel
    kv = torch.zeros(1, 64, 576, device=dev, dtype=torch.bfloat16)
    idx = torch.zeros(1, 8, device=dev, dtype=torch.int32)
    out = torch.zeros(1, 48, 512, device=dev, dtype=torch.bfloat16)
    ws = torch.empty(1 << 20, device=dev, dtype=torch.uint8)
    with pytest.raises(capi.LaunchRejected, match='unsupported shape'):
        capi.sparse_mla_decode_launch(out, q, kv, idx, ws)
    q = torch.zeros(1, 128, 576, device=dev, dtype=torch.bfloat16)
    out = torch.zeros(1, 128, 512, device=dev, dtype=torch.bfloat16)
    with pytest.raises(capi.LaunchRejected, match='workspace too small'):
        capi.sparse_mla_decode_launch(out, q, kv, idx, ws[:64])


@pytest.mark.parametrize('ws_config', ['small', '3'])
def test_workspace_verification_flow(ws_config):
    """`python3 -m utils.verification` from inside the workspace, as its user runs it."""
    ws = Path(__file__).resolve().parent.parent / 'cuda-agent_amd' / 'workspaces' / 'sparse_mla'
    assert (ws / 'cuda_extension.so').exists(), 'workspace extension not built'
    env = dict(os.environ, MLA_CONFIG=ws_config)
    out = subprocess.run([sys.executable, '-m', 'utils.verification'], cwd=ws, env=env,
                         capture_output=True, text=True, timeout=900)
    assert out.returncode == 0, out.stdout + out.stderr
    assert '[PASS] check 5/5' in out.stdout and '[PASS] verify success' in out.stdout
