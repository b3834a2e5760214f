"""MI355X-native operators behind the CUDA-Agent workspace interface.

``csrc/``        hand-written gfx950 HIP kernels and their ``extern "C"`` launchers
``lib/``         the built C-ABI library (``libcuda_agent_amd.so``; built by ``build.py``)
``capi.py``      ctypes view of that library, for callers without a compiled binding
``workspaces/``  one reference-shaped workspace per operator (``model.py`` / ``model_new.py`` /
                 ``binding.cpp`` / ``kernels/`` / ``utils/``)

The directory name is not an identifier, so the package is imported under the name
``cuda_agent_amd`` by a loader that points ``importlib`` at this file.
"""

from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent
CSRC_DIR = PACKAGE_DIR / 'csrc'
LIB_DIR = PACKAGE_DIR / 'lib'
WORKSPACES_DIR = PACKAGE_DIR / 'workspaces'
CAPI_LIBRARY = LIB_DIR / 'libcuda_agent_amd.so'
WORKSPACES = ('axpby', 'gdn_decode', 'moe_fp8', 'sparse_mla')
