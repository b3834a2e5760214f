"""CPU checks of the drop-in boundary: the C-ABI library exports what include/*.h declares, the
ctypes table matches the header, the workspaces share identical infrastructure files, and the
harness helpers behave like the reference workspace's (agent_workdir/utils/verification.py:22-62)."""
import ctypes
import importlib
import re
import subprocess
import sys
from pathlib import Path

import pytest
import torch

REPO = Path(__file__).resolve().parent.parent
HEADER = REPO / 'include' / 'cuda_agent_amd.h'
PKG = REPO / 'cuda-agent_amd'
WORKSPACES = ['axpby', 'gdn_decode', 'moe_fp8', 'sparse_mla']
INFRA = ['binding.cpp', 'binding_registry.h', 'utils/__init__.py', 'utils/compile.py',
         'utils/compile.sh', 'utils/verification.py', 'utils/profiling.py',
         'kernels/launch_status.hip']


def declared_functions():
    text = re.sub(r'/\*.*?\*/', '', HEADER.read_text(), flags=re.S)
    text = text.split('extern "C" {', 1)[1]
    decls = re.findall(r'\b(?:void|int|size_t|long)\s+(\w+)\s*\(([^;{]*?)\)\s*;', text, flags=re.S)
    return {name: [a.strip() for a in args.split(',')] if args.strip() != 'void' else []
            for name, args in decls}


def test_header_declares_the_launchers():
    names = set(declared_functions())
    assert {'axpby_launcher', 'gdn_decode_launcher', 'cuda_agent_amd_last_status'} <= names


def test_library_exports_every_declared_symbol():
    from cuda_agent_amd import CAPI_LIBRARY
    assert CAPI_LIBRARY.exists(), 'build the library first: python __graft_entry__.py'
    lib = ctypes.CDLL(str(CAPI_LIBRARY))
    for name in declared_functions():
        assert hasattr(lib, name), f'{name} is declared in the header but not exported'


def test_ctypes_table_matches_header():
    from cuda_agent_amd import capi
    decls = declared_functions()
    assert set(capi.SIGNATURES) == set(decls)
    for name, args in decls.items():
        assert len(capi.SIGNATURES[name][1]) == len(args), name
        for ctype, arg in zip(capi.SIGNATURES[name][1], args):
            if '*' in arg or 'hipStream_t' in arg:
                assert ctype is ctypes.c_void_p, (name, arg)
            elif arg.startswith('float'):
                assert ctype is ctypes.c_float, (name, arg)
            elif arg.startswith('size_t'):
                assert ctype is ctypes.c_size_t, (name, arg)
            elif arg.startswith('int'):
                assert ctype is ctypes.c_int, (name, arg)


def test_library_has_no_torch_dependency():
    from cuda_agent_amd import CAPI_LIBRARY
    out = subprocess.run(['readelf', '-d', str(CAPI_LIBRARY)], capture_output=True, text=True).stdout
    needed = ' '.join(line for line in out.splitlines() if 'NEEDED' in line)
    assert 'libamdhip64' in needed
    assert 'torch' not in needed and 'c10' not in needed and 'python' not in needed


def test_status_word_starts_clear(capi):
    assert capi.library().cuda_agent_amd_last_status() == 0


def test_rejected_launch_sets_status_without_touching_the_gpu(capi):
    lib = capi.library()
    # dk = 64 has no kernel: rejected on the host before any HIP call
    lib.gdn_decode_launcher(None, None, None, None, None, None, None, 1, 2, 2, 64, 128, 0, 0, None)
    assert lib.cuda_agent_amd_last_status() == 1
    assert lib.cuda_agent_amd_last_status() == 0
    lib.gdn_decode_launcher(None, None, None, None, None, None, None, 1, 2, 2, 128, 128, 0, 0, None)
    assert lib.cuda_agent_amd_last_status() == 2
    # empty problems are silent no-ops (agent_workdir/kernels/axpby.cu:21)
    lib.axpby_launcher(None, None, None, 1.0, 0, 0, None)
    lib.gdn_decode_launcher(None, None, None, None, None, None, None, 0, 2, 2, 128, 128, 0, 0, None)
    assert lib.cuda_agent_amd_last_status() == 0


@pytest.mark.parametrize('rel', INFRA)
def test_workspaces_share_identical_infrastructure(rel):
    blobs = {(PKG / 'workspaces' / w / rel).read_bytes() for w in WORKSPACES}
    assert len(blobs) == 1, f'{rel} differs between workspaces'


@pytest.mark.parametrize('ws', WORKSPACES)
def test_workspace_layout(ws):
    root = PKG / 'workspaces' / ws
    if not (root / 'model_new.py').exists():
        pytest.skip(f'{ws} workspace not populated yet')
    for rel in ['model.py', 'model_new.py', 'binding.cpp', 'binding_registry.h', 'kernels']:
        assert (root / rel).exists(), rel
    hips = sorted(p.name for p in (root / 'kernels').glob('*.hip'))
    bindings = sorted(p.name for p in (root / 'kernels').glob('*_binding.cpp'))
    assert hips and bindings
    for src in (root / 'kernels').glob('*.hip'):
        assert '#include <torch' not in src.read_text(), 'kernel sources include no torch header'
    for src in (PKG / 'csrc').glob('*'):
        text = src.read_text()
        assert '#include <torch' not in text and 'cuda_runtime' not in text, src.name


def _workspace_module(ws, name):
    """Import utils.<name> of a workspace the way `python3 -m utils.<name>` does (cwd = workspace)."""
    root = PKG / 'workspaces' / ws
    if not (root / 'cuda_extension.so').exists():
        pytest.skip('workspace extension not built')
    for mod in ['model', 'model_new', 'cuda_extension', 'utils', f'utils.{name}']:
        sys.modules.pop(mod, None)
    sys.path.insert(0, str(root))
    try:
        return importlib.import_module(f'utils.{name}')
    finally:
        sys.path.remove(str(root))
        for mod in ['model', 'model_new', 'utils']:
            sys.modules.pop(mod, None)


def test_extension_registers_its_operator():
    _workspace_module('axpby', 'verification')
    ext = sys.modules['cuda_extension']
    assert ext.registered_bindings() == ['axpby']
    assert 'config' in ext.axpby_forward.__doc__
    with pytest.raises(RuntimeError, match='must be a GPU tensor'):
        ext.axpby_forward(torch.zeros(4), torch.zeros(4), 2.0, 0)


def test_check_equal_semantics():
    v = _workspace_module('axpby', 'verification')
    a = torch.arange(6.0).reshape(2, 3)
    v.check_equal(a, a + 5e-3)                       # inside atol=1e-2
    v.check_equal((a, [a, 3]), (a.clone(), [a.clone(), 3]))
    v.check_equal({'x': a, 'extra': 1}, {'x': a})    # only the expected keys are looked up
    with pytest.raises(AssertionError):
        v.check_equal(a, a + 1.0)
    with pytest.raises(AssertionError):
        v.check_equal((a,), [a])                     # tuple vs list is a type mismatch
    with pytest.raises(AssertionError):
        v.check_equal([a], [a, a])
    with pytest.raises(AssertionError):
        v.check_equal(a, a.double())                 # assert_close checks dtype
    with pytest.raises(AssertionError):
        v.check_equal(3, 4)
    with pytest.raises(TypeError):
        v.check_equal(None, None)


def test_transform_tensors_turns_tuples_into_lists():
    v = _workspace_module('axpby', 'verification')
    a = torch.ones(2)
    out = v.transform_tensors((a, {'k': (a, 'txt')}, 7), lambda t: t * 2)
    assert isinstance(out, list) and isinstance(out[1]['k'], list)
    assert torch.equal(out[0], a * 2) and out[1]['k'][1] == 'txt' and out[2] == 7


def test_functional_namespace_is_blocked_and_restored():
    import torch.nn.functional as F
    v = _workspace_module('axpby', 'verification')
    before = F.relu
    with v.block_torch_functional():
        with pytest.raises(RuntimeError, match='torch.nn.functional.relu is not allowed'):
            F.relu(torch.zeros(1))
        with pytest.raises(RuntimeError, match='softplus'):
            F.softplus(torch.zeros(1))
        torch.relu(torch.zeros(1))                   # torch.* itself is not blocked
    assert F.relu is before
    with pytest.raises(ValueError):
        with v.block_torch_functional(excludes={'relu'}):
            assert F.relu is before                  # excluded names keep their function
            raise ValueError('restored on exceptions too')
    assert F.relu is before and F.softplus(torch.zeros(1)).item() > 0


def test_profiling_cli_defaults():
    p = _workspace_module('axpby', 'profiling')
    args = p.parse_args([])
    assert args.iters == 10 and args.single_run is None and p.WARMUP_ITERS == 5
    args = p.parse_args(['--iters', '3', '--single-run', 'cuda_extension'])
    assert args.iters == 3 and args.single_run == 'cuda_extension'


def test_compile_finds_hip_and_cpp_sources(tmp_path, monkeypatch):
    sys.path.insert(0, str(PKG / 'workspaces' / 'axpby'))
    try:
        sys.modules.pop('utils', None)
        comp = importlib.import_module('utils.compile')
    finally:
        sys.path.pop(0)
        sys.modules.pop('utils', None)
        sys.modules.pop('utils.compile', None)
    monkeypatch.chdir(tmp_path)
    assert comp.compile_kernels() == 1               # no sources -> rc 1
    (tmp_path / 'kernels').mkdir()
    for rel in ['binding.cpp', 'kernels/b.hip', 'kernels/a_binding.cpp', 'kernels/skip.cu', 'notes.txt']:
        (tmp_path / rel).write_text('')
    assert comp.find_sources() == ['binding.cpp', 'kernels/a_binding.cpp', 'kernels/b.hip']


def test_compile_failure_reports_rc1(tmp_path, monkeypatch, capsys):
    sys.path.insert(0, str(PKG / 'workspaces' / 'axpby'))
    try:
        sys.modules.pop('utils', None)
        comp = importlib.import_module('utils.compile')
    finally:
        sys.path.pop(0)
        sys.modules.pop('utils', None)
        sys.modules.pop('utils.compile', None)
    monkeypatch.chdir(tmp_path)
    (tmp_path / 'broken.hip').write_text('this is not HIP\n')
    assert comp.compile_kernels() == 1
    out = capsys.readouterr().out
    assert 'Compiling 1 files: broken.hip' in out and 'Compilation failed.' in out
    assert not (tmp_path / 'cuda_extension.so').exists()
