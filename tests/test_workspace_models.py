"""The eager `Model` of every operator workspace is the reference its verification flow uses;
these CPU tests tie each of them to the oracle (same inputs, same results), check the input
factories against the workload definition, and check the model contract
(agent_workdir/model.py:9-26, agent_workdir/model_new.py:6-13: same constructor arguments, same
state_dict keys)."""
import importlib.util
import os
import re
import sys
from pathlib import Path

import pytest
import torch

from oracle import gdn, mla, moe

WS = Path(__file__).resolve().parent.parent / 'cuda-agent_amd' / 'workspaces'


def load_model_module(workspace, **env):
    old = {k: os.environ.get(k) for k in env}
    os.environ.update(env)
    try:
        spec = importlib.util.spec_from_file_location(f'{workspace}_model_{abs(hash(tuple(env.items())))}',
                                                      WS / workspace / 'model.py')
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        return mod
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def test_gdn_model_is_the_oracle():
    m = load_model_module('gdn_decode', GDN_CONFIG='0')
    model = m.Model(*m.get_init_inputs())
    ins = m.get_inputs()
    assert [tuple(t.shape) for t in ins] == [(1, 16, 128), (1, 16, 128), (1, 16, 128), (1, 16), (1, 16),
                                             (1, 16, 128, 128)]
    assert all(t.dtype == torch.float32 for t in ins)
    want_o, want_s = gdn.gdn_decode_step(*ins[:5], ins[5].clone())
    state = ins[5].clone()
    out = model(*ins[:5], state)
    assert isinstance(out, tuple) and out[1] is state
    torch.testing.assert_close(out[0], want_o, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(out[1], want_s, rtol=1e-5, atol=1e-7)
    again = m.get_inputs()
    assert not torch.equal(again[0], ins[0])            # a new draw each call


def test_gdn_batched_config_shapes():
    m = load_model_module('gdn_decode', GDN_CONFIG='1')
    c = m.CONFIGS[1]
    assert (c['batch'], c['n_v_heads'], c['n_qk_heads'], c['qkv_dtype']) == (256, 32, 16, torch.bfloat16)
    assert m.get_init_inputs() == [32, 16, 128, 128]
    assert 256 * 32 * 128 * 128 * 4 == 536870912         # the 537 MB state of the workload


def test_mla_model_is_the_oracle():
    m = load_model_module('sparse_mla', MLA_CONFIG='small')
    model = m.Model(*m.get_init_inputs())
    q, kv, idx = m.get_inputs()
    assert q.shape == (4, 128, 576) and kv.shape == (4, 4096, 576) and idx.shape == (4, 512)
    assert q.dtype == kv.dtype == torch.bfloat16 and idx.dtype == torch.int32
    for b in range(4):
        assert len(set(idx[b].tolist())) == 512
    out = model(q, kv, idx)
    want = mla.sparse_mla_decode(q, kv, idx)
    assert out.dtype == torch.bfloat16 and out.shape == (4, 128, 512)
    assert mla.rel_rms_error(out.float(), want.float()) < 2e-2   # both bf16; fp32 summation order
    assert m.CONFIGS['3'] == dict(batch=64, n_heads=128, n_kv_rows=32768, topk=2048)
    padded = idx.clone()
    padded[:, ::7] = -1
    torch.testing.assert_close(model(q, kv, padded).float(), mla.sparse_mla_decode(q, kv, padded).float(),
                               rtol=2e-2, atol=2e-2)


def test_moe_model_is_the_oracle():
    m = load_model_module('moe_fp8', MOE_CONFIG='small')
    model = m.Model(*m.get_init_inputs())
    assert set(model.state_dict()) == {'w13_q', 'w13_s', 'w2_q', 'w2_s'}
    assert model.w13_q.dtype == torch.float8_e4m3fn and model.w13_q.shape == (32, 1024, 1024)
    assert ((model.w13_q.view(torch.uint8) & 0x7F) != 0x7F).all()      # no NaN codes
    assert model.w13_s.min() >= 0.5 / 448 - 1e-9 and model.w13_s.max() <= 1.5 / 448 + 1e-9
    x, logits = m.get_inputs()
    assert x.dtype == torch.bfloat16 and x.shape == (64, 1024) and logits.shape == (64, 32)
    out = model(x, logits)
    want = moe.moe_forward(x, logits, model.w13_q, model.w13_s, model.w2_q, model.w2_s, top_k=8)
    assert out.dtype == torch.bfloat16
    assert torch.equal(out, want)                       # the same arithmetic, statement by statement


def test_moe_prefill_config_biases_sixteen_experts():
    m = load_model_module('moe_fp8', MOE_CONFIG='4')
    assert m.CONFIGS['4'] == dict(tokens=8192, hidden=7168, inter=2048, n_experts=256, top_k=8, biased=16)
    assert m.CONFIGS['2'] == dict(tokens=64, hidden=7168, inter=2048, n_experts=256, top_k=8, biased=0)
    m.CONFIGS['4'].update(hidden=128)                    # shrink the draw, keep tokens and experts
    x, logits = m.get_inputs()
    mean = logits.mean(0)
    assert int((mean > 1.0).sum()) == 16                 # +2 on 16 experts, the rest around 0
    x2, logits2 = m.get_inputs()
    assert torch.equal(logits2.mean(0) > 1.0, mean > 1.0)  # the same 16 on every draw


@pytest.mark.parametrize('workspace', ['axpby', 'gdn_decode', 'sparse_mla', 'moe_fp8'])
def test_model_new_mirrors_model_constructor(workspace):
    src = (WS / workspace / 'model.py').read_text()
    new = (WS / workspace / 'model_new.py').read_text()
    sig = re.search(r'class Model\(nn.Module\):.*?def __init__\(self, (.*?)\) -> None', src, re.S).group(1)
    sig_new = re.search(r'class ModelNew\(nn.Module\):.*?def __init__\(self, (.*?)\) -> None', new, re.S).group(1)
    assert sig == sig_new
    assert 'import cuda_extension' in new
    assert 'torch.nn.functional' not in new and 'F.' not in new
    assert set(re.findall(r"register_buffer\('(\w+)'", src)) == set(re.findall(r"register_buffer\('(\w+)'", new))
