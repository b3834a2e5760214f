"""GPU check of the smoke operator through the C ABI and through its workspace flow."""
import subprocess
import sys
from pathlib import Path

import pytest
import torch

pytestmark = pytest.mark.gpu
REPO = Path(__file__).resolve().parent.parent


@pytest.mark.parametrize('config', [0, 1, 2])
@pytest.mark.parametrize('n', [1, 3, 128, 1000003])
def test_axpby_bit_exact(capi, dev, n, config):
    gen = torch.Generator().manual_seed(n)
    a = torch.randn(n, generator=gen).to(dev)
    b = torch.randn(n, generator=gen).to(dev)
    out = torch.empty_like(a)
    capi.axpby_launch(out, a, b, 2.0, config=config)
    # alpha = 2 makes alpha*a exact, so fused and unfused multiply-add agree bit for bit
    assert torch.equal(out, 2.0 * a + b)


def test_axpby_unaligned_views(capi, dev):
    base = torch.randn(4099, device=dev)
    a, b = base[1:4098].contiguous(), base[2:4099].contiguous()
    a_un = torch.empty(4098, device=dev)[1:]
    a_un.copy_(a)                        # base pointer 4 bytes past a 16-byte boundary
    out = torch.empty_like(a)
    capi.axpby_launch(out, a_un, b, 2.0)
    assert torch.equal(out, 2.0 * a + b)


def test_workspace_flow():
    ws = REPO / 'cuda-agent_amd' / 'workspaces' / 'axpby'
    assert (ws / 'cuda_extension.so').exists(), 'workspace extension not built'
    out = subprocess.run([sys.executable, '-m', 'utils.verification'], cwd=ws, capture_output=True,
                         text=True, timeout=300)
    assert out.returncode == 0 and '[PASS] verify success' in out.stdout, out.stdout + out.stderr
    out = subprocess.run([sys.executable, '-m', 'utils.profiling', '--single-run', 'cuda_extension'],
                         cwd=ws, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and '[DONE] single-run completed' in out.stdout, out.stdout + out.stderr
