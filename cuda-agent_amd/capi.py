"""ctypes view of ``lib/libcuda_agent_amd.so`` (the C ABI declared in ``include/cuda_agent_amd.h``).

The library is loaded on first use and never built here. A missing library, a missing symbol or
a launch the library rejects raises: there is no fallback path.

The ``*_launch`` helpers take torch tensors only to read their device pointers and shapes;
every output and scratch buffer is allocated by the caller, as the launcher ABI requires.
"""

import ctypes
from ctypes import c_float, c_int, c_size_t, c_void_p

from . import CAPI_LIBRARY

_P = c_void_p

# name -> (restype, argtypes); mirrors include/cuda_agent_amd.h declaration by declaration
SIGNATURES = {
    'cuda_agent_amd_last_status': (c_int, []),
    'axpby_launcher': (None, [_P, _P, _P, c_float, c_int, c_int, _P]),
    'gdn_decode_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int,
                                   c_int, c_int, _P]),
    'sparse_mla_decode_launcher': (None, [_P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int,
                                          c_int, c_int, c_float, c_int, c_int, _P]),
    'sparse_mla_decode_num_splits': (c_int, [c_int, c_int, c_int, c_int]),
    'sparse_mla_decode_workspace_bytes': (c_size_t, [c_int, c_int, c_int, c_int]),
}

STATUS_NAMES = {0: 'ok', 1: 'unsupported shape', 2: 'bad argument', 3: 'workspace too small'}

_lib = None


class LaunchRejected(RuntimeError):
    pass


def library():
    """The loaded C-ABI library with argument types set on every declared entry point."""
    global _lib
    if _lib is None:
        if not CAPI_LIBRARY.exists():
            raise RuntimeError(
                f'{CAPI_LIBRARY} is not built; run `python __graft_entry__.py` '
                '(or cuda-agent_amd/build.py) first')
        import torch  # noqa: F401  (its HIP runtime must be the one in the process)
        lib = ctypes.CDLL(str(CAPI_LIBRARY))
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check_status(what):
    code = library().cuda_agent_amd_last_status()
    if code != 0:
        raise LaunchRejected(f'{what}: launch rejected ({STATUS_NAMES.get(code, code)})')


def _ptr(t):
    return c_void_p(t.data_ptr())


def _stream(stream=None):
    import torch
    s = torch.cuda.current_stream() if stream is None else stream
    return c_void_p(s.cuda_stream)


def _require(cond, msg):
    if not cond:
        raise ValueError(msg)


def _device_contiguous(**tensors):
    for name, t in tensors.items():
        _require(t.is_cuda, f'{name} must be a GPU tensor')
        _require(t.is_contiguous(), f'{name} must be contiguous')


def axpby_launch(out, a, b, alpha, config=0, stream=None):
    import torch
    _device_contiguous(out=out, a=a, b=b)
    _require(out.dtype == a.dtype == b.dtype == torch.float32, 'axpby: fp32 only')
    _require(out.shape == a.shape == b.shape, 'axpby: shapes differ')
    library().axpby_launcher(_ptr(out), _ptr(a), _ptr(b), float(alpha), a.numel(), config,
                             _stream(stream))
    check_status('axpby_launcher')
    return out


def gdn_decode_launch(o, state, q, k, v, g, beta, config=0, stream=None):
    """One decode step; ``state`` is updated in place and ``o`` written."""
    import torch
    _device_contiguous(o=o, state=state, q=q, k=k, v=v, g=g, beta=beta)
    B, Hv, dk, dv = state.shape
    Hqk = q.shape[1]
    _require(state.dtype == o.dtype == g.dtype == beta.dtype == torch.float32,
             'gdn_decode: o, state, g, beta must be fp32')
    _require(q.dtype == k.dtype == v.dtype and q.dtype in (torch.float32, torch.bfloat16),
             'gdn_decode: q, k, v must share dtype fp32 or bf16')
    _require(tuple(q.shape) == (B, Hqk, dk) and tuple(k.shape) == (B, Hqk, dk), 'gdn_decode: q/k shape')
    _require(tuple(v.shape) == (B, Hv, dv) and tuple(o.shape) == (B, Hv, dv), 'gdn_decode: v/o shape')
    _require(tuple(g.shape) == (B, Hv) and tuple(beta.shape) == (B, Hv), 'gdn_decode: g/beta shape')
    library().gdn_decode_launcher(_ptr(o), _ptr(state), _ptr(q), _ptr(k), _ptr(v), _ptr(g),
                                  _ptr(beta), B, Hv, Hqk, dk, dv,
                                  0 if q.dtype == torch.float32 else 1, config, _stream(stream))
    check_status('gdn_decode_launcher')
    return o, state


def sparse_mla_workspace_bytes(batch, n_heads, topk, config=0):
    return int(library().sparse_mla_decode_workspace_bytes(batch, n_heads, topk, config))


def sparse_mla_decode_launch(out, q, kv, idx, workspace, sm_scale=192 ** -0.5, config=0, stream=None):
    """out [B,H,512] (bf16, or fp32 for the unrounded values) <- attention of q [B,H,576] over rows idx [B,topk] of kv [B,N,576].
    ``workspace`` is a uint8 device tensor of at least ``sparse_mla_workspace_bytes`` bytes."""
    import torch
    _device_contiguous(out=out, q=q, kv=kv, idx=idx, workspace=workspace)
    B, H, d_qk = q.shape
    N = kv.shape[1]
    topk = idx.shape[1]
    d_v = out.shape[2]
    _require(q.dtype == kv.dtype == torch.bfloat16, 'sparse_mla: q, kv must be bf16')
    _require(out.dtype in (torch.bfloat16, torch.float32), 'sparse_mla: out must be bf16 or fp32')
    _require(idx.dtype == torch.int32, 'sparse_mla: idx must be int32')
    _require(tuple(kv.shape) == (B, N, d_qk) and tuple(idx.shape) == (B, topk), 'sparse_mla: kv/idx shape')
    _require(tuple(out.shape) == (B, H, d_v), 'sparse_mla: out shape')
    library().sparse_mla_decode_launcher(_ptr(out), _ptr(q), _ptr(kv), _ptr(idx), _ptr(workspace),
                                         workspace.numel() * workspace.element_size(), B, H, N, topk,
                                         d_qk, d_v, float(sm_scale),
                                         0 if out.dtype == torch.bfloat16 else 1, config,
                                         _stream(stream))
    check_status('sparse_mla_decode_launcher')
    return out
