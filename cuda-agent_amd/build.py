"""Build steps: the torch-free C-ABI library from ``csrc/`` and every workspace extension.

``build_capi()`` compiles each ``csrc/*.hip`` with ``hipcc --offload-arch=gfx950`` and links
``lib/libcuda_agent_amd.so``. ``build_workspace(name)`` runs the workspace's own
``python3 -m utils.compile`` from inside it, exactly as a user of the workspace would.
"""

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
CSRC_DIR = PACKAGE_DIR / 'csrc'
LIB_DIR = PACKAGE_DIR / 'lib'
WORKSPACES_DIR = PACKAGE_DIR / 'workspaces'

GPU_ARCH = 'gfx950'
DEVICE_FLAGS = [
    '-Wno-inline-asm',
    '-O3', '-std=c++17', '-fPIC', f'--offload-arch={GPU_ARCH}', '-fno-gpu-rdc',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
]


def _hipcc() -> str:
    rocm = os.environ.get('ROCM_PATH') or os.environ.get('ROCM_HOME') or '/opt/rocm'
    return shutil.which('hipcc') or f'{rocm}/bin/hipcc'


def _run(cmd, cwd=None):
    proc = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f'command failed ({proc.returncode}): {" ".join(map(str, cmd))}\n{proc.stdout}')
    return proc.stdout


def _jobs(n):
    return max(1, min(n, int(os.environ.get('MAX_JOBS', os.cpu_count() or 1))))


def build_capi(verbose=False) -> Path:
    sources = sorted(CSRC_DIR.glob('*.hip'))
    if not sources:
        raise RuntimeError(f'no HIP sources under {CSRC_DIR}')
    obj_dir = LIB_DIR / 'obj'
    if obj_dir.exists():
        shutil.rmtree(obj_dir)
    obj_dir.mkdir(parents=True)
    objects = [obj_dir / (src.stem + '.o') for src in sources]
    cmds = [[_hipcc(), *DEVICE_FLAGS, '-c', str(src), '-o', str(obj)]
            for src, obj in zip(sources, objects)]
    with ThreadPoolExecutor(max_workers=_jobs(len(cmds))) as pool:
        list(pool.map(_run, cmds))
    out = LIB_DIR / 'libcuda_agent_amd.so'
    _run([_hipcc(), '-shared', '-fPIC', f'--offload-arch={GPU_ARCH}', '-o', str(out), *map(str, objects)])
    shutil.rmtree(obj_dir)
    if verbose:
        print(f'built {out} from {len(sources)} sources')
    return out


def build_workspace(name: str, verbose=False) -> Path:
    ws = WORKSPACES_DIR / name
    out = _run([sys.executable, '-m', 'utils.compile'], cwd=ws)
    if verbose:
        print(out, end='')
    so = ws / 'cuda_extension.so'
    if not so.exists():
        raise RuntimeError(f'workspace {name}: cuda_extension.so missing after compile\n{out}')
    return so


def build_all(verbose=False):
    from . import WORKSPACES
    build_capi(verbose)
    ready = [w for w in WORKSPACES if (WORKSPACES_DIR / w / 'model_new.py').exists()]
    # each workspace build is itself parallel over its sources; run two at a time
    with ThreadPoolExecutor(max_workers=2) as pool:
        list(pool.map(lambda w: build_workspace(w, verbose), ready))


if __name__ == '__main__':
    import importlib.util
    spec = importlib.util.spec_from_file_location(
        'cuda_agent_amd', PACKAGE_DIR / '__init__.py', submodule_search_locations=[str(PACKAGE_DIR)])
    pkg = importlib.util.module_from_spec(spec)
    sys.modules['cuda_agent_amd'] = pkg
    spec.loader.exec_module(pkg)
    from cuda_agent_amd.build import build_all as _build_all
    _build_all(verbose=True)
