#!/usr/bin/env python3
"""Force-compile the workspace's HIP and C++ sources into ./cuda_extension.so.

Same command, glob rules, log lines and exit codes as the reference workspace's build step
(agent_workdir/utils/compile.py:11-63), with the internals written for ROCm:

* ``*.hip`` files (root and ``kernels/``) hold kernels and their ``extern "C"`` launchers.
  They include no torch header and go straight to ``hipcc --offload-arch=gfx950``; nothing
  is passed through a CUDA-to-HIP source translator.
* ``*.cpp`` files are host-only binding code (pybind11 / libtorch) and go to the host
  compiler with torch's include paths.
* everything is linked into ``build/forced_compile/cuda_extension.so`` and copied to the
  workspace root.

Run from the workspace directory: ``python3 -m utils.compile`` (or ``bash utils/compile.sh``).
"""

import os
import shutil
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

GPU_ARCH = 'gfx950'

HOST_FLAGS = ['-O3', '-std=c++17', '-fPIC']
# Packed-FP32 instruction selection is switched off for every device translation unit.
DEVICE_FLAGS = [
    '-Wno-inline-asm',
    '-O3', '-std=c++17', '-fPIC', f'--offload-arch={GPU_ARCH}', '-fno-gpu-rdc',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
]


def find_sources() -> list[str]:
    root = Path('.')
    kernels_dir = Path('kernels')
    found = set()
    for pattern in ('*.hip', '*.cpp'):
        found.update(str(p) for p in root.glob(pattern))
        if kernels_dir.is_dir():
            found.update(str(p) for p in kernels_dir.glob(pattern))
    return sorted(found)


def _rocm_home() -> str:
    return os.environ.get('ROCM_PATH') or os.environ.get('ROCM_HOME') or '/opt/rocm'


def _host_include_flags() -> list[str]:
    import pybind11
    import torch.utils.cpp_extension as cpp_ext

    dirs = list(cpp_ext.include_paths())
    dirs += [pybind11.get_include(), sysconfig.get_paths()['include'], f'{_rocm_home()}/include']
    flags = []
    for d in dict.fromkeys(dirs):
        flags += ['-isystem', d]
    return flags


def _compile_command(src: str, obj: Path) -> list[str]:
    if src.endswith('.hip'):
        hipcc = shutil.which('hipcc') or f'{_rocm_home()}/bin/hipcc'
        return [hipcc, *DEVICE_FLAGS, '-c', src, '-o', str(obj)]
    cxx = os.environ.get('CXX', 'g++')
    defines = [
        '-D__HIP_PLATFORM_AMD__=1', '-DUSE_ROCM=1', '-DTORCH_EXTENSION_NAME=cuda_extension',
        '-DTORCH_API_INCLUDE_EXTENSION_H',
    ]
    return [cxx, *HOST_FLAGS, *defines, *_host_include_flags(), '-c', src, '-o', str(obj)]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f'command failed ({proc.returncode}): {" ".join(cmd)}\n{proc.stdout}')


def _build(sources: list[str], build_dir: Path) -> Path:
    import torch
    import torch.utils.cpp_extension as cpp_ext

    objects = []
    jobs = []
    for src in sources:
        obj = build_dir / (src.replace('/', '_').replace('.', '_') + '.o')
        objects.append(obj)
        jobs.append(_compile_command(src, obj))
    workers = max(1, min(len(jobs), int(os.environ.get('MAX_JOBS', os.cpu_count() or 1))))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        list(pool.map(_run, jobs))

    torch_lib = os.path.join(os.path.dirname(torch.__file__), 'lib')
    lib_dirs = [torch_lib] + [d for d in cpp_ext.library_paths() if d != torch_lib and os.path.isdir(d)]
    built_so = build_dir / 'cuda_extension.so'
    link = [os.environ.get('CXX', 'g++'), '-shared', '-o', str(built_so), *map(str, objects)]
    for d in lib_dirs:
        link += [f'-L{d}']
    # torch's own copy of the HIP runtime comes first on the search path, so the extension
    # binds to the runtime that torch has already loaded.
    link += [f'-Wl,-rpath,{torch_lib}', '-lc10', '-lc10_hip', '-ltorch_cpu', '-ltorch_hip',
             '-ltorch', '-ltorch_python', '-lamdhip64']
    _run(link)
    return built_so


def compile_kernels() -> int:
    build_dir = Path('build/forced_compile')
    output_so = Path('cuda_extension.so')
    sources = find_sources()

    if not sources:
        print('Error: no source files found (*.hip, *.cpp in root or kernels/)')
        return 1

    print(f'Compiling {len(sources)} files: {", ".join(sources)}')

    if build_dir.exists():
        shutil.rmtree(build_dir)
    build_dir.mkdir(parents=True, exist_ok=True)
    if output_so.exists():
        output_so.unlink()

    try:
        built_so = _build(sources, build_dir)
    except Exception as exc:
        print('Compilation failed.')
        print(str(exc))
        return 1

    if built_so.exists():
        shutil.copy2(built_so, output_so)
        print(f'Compile success: {output_so}')
        return 0

    print('Compilation finished but cuda_extension.so was not generated.')
    return 1


def main() -> int:
    return compile_kernels()


if __name__ == '__main__':
    sys.exit(main())
