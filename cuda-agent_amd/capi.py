"""ctypes view of ``lib/libcuda_agent_amd.so`` (the C ABI declared in ``include/cuda_agent_amd.h``).

The library is loaded on first use and never built here. A missing library, a missing symbol or
a launch the library rejects raises: there is no fallback path.

The ``*_launch`` helpers take torch tensors only to read their device pointers and shapes;
every output and scratch buffer is allocated by the caller, as the launcher ABI requires.
"""

import ctypes
from ctypes import c_float, c_int, c_long, c_size_t, c_void_p

from . import CAPI_LIBRARY

_P = c_void_p

# name -> (restype, argtypes); mirrors include/cuda_agent_amd.h declaration by declaration
SIGNATURES = {
    'cuda_agent_amd_last_status': (c_int, []),
    'axpby_launcher': (None, [_P, _P, _P, c_float, c_int, c_int, _P]),
    'calibrate_mfma_launcher': (None, [_P, _P, c_size_t, _P, _P, c_int, c_int, c_int, _P]),
    'gdn_decode_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int,
                                   c_int, c_int, _P]),
    'gdn_decode_fused_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int,
                                         c_int, c_int, c_int, _P]),
    'gdn_decode_fused_norm_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_float, c_int, c_int,
                                              c_int, c_int, c_int, c_int, c_int, _P]),
    'causal_conv1d_update_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int,
                                             c_int, c_int, c_int, _P]),
    'sparse_mla_decode_launcher': (None, [_P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int,
                                          c_int, c_int, c_float, c_int, c_int, _P]),
    'sparse_mla_decode_paged_launcher': (None, [_P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int,
                                                c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                                _P]),
    'sparse_mla_decode_fp8_paged_launcher': (None, [_P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int,
                                                    c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                                    _P]),
    'sparse_mla_decode_num_splits': (c_int, [c_int, c_int, c_int, c_int]),
    'sparse_mla_decode_workspace_bytes': (c_size_t, [c_int, c_int, c_int, c_int]),
    'sparse_mla_decode_static_scratch_bytes': (c_size_t, []),
    'sparse_mla_decode_static_launcher': (None, [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                                                 c_int, c_int, _P]),
    'mla_latent_quant_launcher': (None, [_P, _P, c_long, c_int, _P]),
    'sparse_mla_decode_fp8_workspace_bytes': (c_size_t, [c_int, c_int, c_int, c_int]),
    'sparse_mla_decode_fp8_launcher': (None, [_P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int, c_int, c_int,
                                              c_float, c_int, c_int, _P]),
    'mla_index_scores_launcher': (None, [_P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_float, c_int, _P]),
    'mla_index_scores_paged_launcher': (None, [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int,
                                               c_float, c_int, _P]),
    'mla_index_scores_fp8_launcher': (None, [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_float, c_int, _P]),
    'mla_index_scores_fp8_paged_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int,
                                                   c_int, c_float, c_int, _P]),
    'topk_select_launcher': (None, [_P, _P, _P, c_int, c_int, c_int, c_int, _P]),
    'moe_route_launcher': (None, [_P, _P, _P, c_int, c_int, c_int, c_int, _P]),
    'moe_router_logits_num_splits': (c_int, [c_int, c_int, c_int]),
    'moe_router_logits_workspace_bytes': (c_size_t, [c_int, c_int, c_int]),
    'moe_router_logits_launcher': (None, [_P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int, c_int, _P]),
    'moe_router_split_weight_launcher': (None, [_P, _P, c_int, c_int, _P]),
    'moe_router_logits_split_launcher': (None, [_P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int, _P]),
    'moe_route_grouped_launcher': (None, [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                                          c_int, _P]),
    'moe_sort_launcher': (None, [_P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P]),
    'moe_route_sort_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P]),
    'moe_quant_bf16_launcher': (None, [_P, _P, _P, c_int, c_int, c_int, _P]),
    'moe_rmsnorm_quant_launcher': (None, [_P, _P, _P, _P, _P, c_float, c_int, c_int, c_int, _P]),
    'moe_gate_up_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int,
                                    c_int, _P]),
    'moe_down_launcher': (None, [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, _P]),
    'moe_combine_launcher': (None, [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P]),
    'moe_combine_shared_launcher': (None, [_P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P]),
    'moe_fp8_shared_workspace_bytes': (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    'moe_fp8_shared_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int,
                                       c_int, c_int, c_int, c_int, c_int, c_int, _P]),
    'moe_fp8_fused_shared_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int,
                                             c_int, c_int, c_int, c_int, _P]),
    'moe_fp8_workspace_bytes': (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    'moe_fp8_workspace_layout': (c_int, [_P, c_int, c_int, c_int, c_int, c_int, c_int]),
    'moe_fp8_uses_tiled_gemms': (c_int, [c_int, c_int, c_int, c_int, c_int, c_int]),
    'moe_fp8_launcher': (None, [_P, _P, _P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int,
                                c_int, c_int, c_int, _P]),
}

STATUS_NAMES = {0: 'ok', 1: 'unsupported shape', 2: 'bad argument', 3: 'workspace too small',
                4: 'more scratch needed than the static array holds', 5: 'HIP runtime error during set-up'}

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


def calibrate_mfma(seconds=0.25, stream_bytes=0, bf16=False, n_cus=256):
    """Sustained rate of the matrix cores on random operands, alone or beside an HBM stream: launches the
    calibration kernel back to back for about ``seconds`` and returns (PFLOP/s over the MFMA loops of the last
    half of the launches, TB/s streamed beside them, mean kernel time in ms)."""
    import time
    import torch
    dev = torch.device('cuda:0')
    gen = torch.Generator(device=dev).manual_seed(20270)
    if bf16:
        operands = torch.randn(n_cus * 16384 // 2, device=dev, generator=gen).bfloat16()
    else:
        operands = (torch.randn(n_cus * 16384, device=dev, generator=gen) * 40).clamp(-448, 448).to(torch.float8_e4m3fn)
    src = torch.empty(stream_bytes // 4, dtype=torch.int32, device=dev).random_(generator=gen) if stream_bytes else None
    result = torch.zeros(n_cus, 2, dtype=torch.int64, device=dev)
    sink = torch.zeros(2, device=dev)
    iters = 4096
    flops_per_cu = 4 * iters * 4 * 2 * 32 * 32 * (16 if bf16 else 64)

    def launch():
        library().calibrate_mfma_launcher(_ptr(operands), _ptr(src) if src is not None else c_void_p(None), stream_bytes,
                                          _ptr(result), _ptr(sink), n_cus, iters, 1 if bf16 else 0, _stream(None))
        check_status('calibrate_mfma_launcher')

    t0 = time.perf_counter()
    rates, streamed, times = [], [], []
    while time.perf_counter() - t0 < seconds or len(rates) < 4:
        result.zero_()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        launch()
        b.record()
        torch.cuda.synchronize()
        ticks = result[:, 0].double()
        rates.append(flops_per_cu * n_cus / (ticks.mean().item() * 1e-8) / 1e15)
        streamed.append(result[:, 1].sum().item() / (ticks.mean().item() * 1e-8) / 1e12)
        times.append(a.elapsed_time(b))
    half = len(rates) // 2
    mean = lambda v: sum(v[half:]) / len(v[half:])
    return mean(rates), mean(streamed), mean(times)


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


def gdn_decode_fused_launch(o, state, q, k, v, a, b, a_log, dt_bias, config=0, stream=None):
    """One decode step from unnormalised q/k and the gate inputs (see the header); ``state`` is
    updated in place and ``o`` written."""
    import torch
    _device_contiguous(o=o, state=state, q=q, k=k, v=v, a=a, b=b, a_log=a_log, dt_bias=dt_bias)
    B, Hv, dk, dv = state.shape
    Hqk = q.shape[1]
    _require(all(t.dtype == torch.float32 for t in (state, o, a, b, a_log, dt_bias)),
             'gdn_decode_fused: o, state, a, b, a_log, dt_bias must be fp32')
    _require(q.dtype == k.dtype == v.dtype and q.dtype in (torch.float32, torch.bfloat16),
             'gdn_decode_fused: q, k, v must share dtype fp32 or bf16')
    _require(tuple(q.shape) == (B, Hqk, dk) and tuple(k.shape) == (B, Hqk, dk), 'gdn_decode_fused: q/k shape')
    _require(tuple(v.shape) == (B, Hv, dv) and tuple(o.shape) == (B, Hv, dv), 'gdn_decode_fused: v/o shape')
    _require(tuple(a.shape) == (B, Hv) and tuple(b.shape) == (B, Hv), 'gdn_decode_fused: a/b shape')
    _require(tuple(a_log.shape) == (Hv,) and tuple(dt_bias.shape) == (Hv,), 'gdn_decode_fused: a_log/dt_bias shape')
    library().gdn_decode_fused_launcher(_ptr(o), _ptr(state), _ptr(q), _ptr(k), _ptr(v), _ptr(a), _ptr(b),
                                        _ptr(a_log), _ptr(dt_bias), B, Hv, Hqk, dk, dv,
                                        0 if q.dtype == torch.float32 else 1, config, _stream(stream))
    check_status('gdn_decode_fused_launcher')
    return o, state


def gdn_decode_fused_norm_launch(out, state, q, k, v, a, b, a_log, dt_bias, z, norm_w, eps=1e-6, config=0,
                                 stream=None):
    """The fused step plus the gated RMS normalisation of its read-out: out [B,Hv,128] (dtype of q/k/v) =
    norm_w * o * rsqrt(mean(o^2) + eps) * silu(z); state updated in place."""
    import torch
    _device_contiguous(out=out, state=state, q=q, k=k, v=v, a=a, b=b, a_log=a_log, dt_bias=dt_bias, z=z,
                       norm_w=norm_w)
    B, Hv, dk, dv = state.shape
    Hqk = q.shape[1]
    _require(state.dtype == torch.float32, 'gdn_decode: state must be fp32')
    _require(q.dtype == k.dtype == v.dtype == z.dtype == norm_w.dtype == out.dtype
             and q.dtype in (torch.float32, torch.bfloat16), 'gdn_decode: q, k, v, z, norm_w, out of one type')
    _require(all(t.dtype == torch.float32 for t in (a, b, a_log, dt_bias)), 'gdn_decode: gate tensors must be fp32')
    _require(tuple(q.shape) == tuple(k.shape) == (B, Hqk, dk) and tuple(v.shape) == (B, Hv, dv), 'gdn_decode: q/k/v')
    _require(tuple(z.shape) == tuple(out.shape) == (B, Hv, dv) and tuple(norm_w.shape) == (dv,),
             'gdn_decode: z/out [B,Hv,dv], norm_w [dv]')
    _require(tuple(a.shape) == tuple(b.shape) == (B, Hv) and tuple(a_log.shape) == tuple(dt_bias.shape) == (Hv,),
             'gdn_decode: gate shapes')
    library().gdn_decode_fused_norm_launcher(
        _ptr(out), _ptr(state), _ptr(q), _ptr(k), _ptr(v), _ptr(a), _ptr(b), _ptr(a_log), _ptr(dt_bias), _ptr(z),
        _ptr(norm_w), float(eps), B, Hv, Hqk, dk, dv, 0 if q.dtype == torch.float32 else 1, config,
        _stream(stream))
    check_status('gdn_decode_fused_norm_launcher')
    return out, state


def causal_conv1d_update_launch(q_out, k_out, v_out, conv_state, x, weight, bias=None, activation='silu',
                                config=0, stream=None):
    """conv_state [B,C,L] shifted in place by x [B,C]; q_out [B,key_dim], k_out [B,key_dim],
    v_out [B,C-2*key_dim] <- activation(bias + the K newest values . weight [C,K]).
    q_out = k_out = None puts every channel into v_out."""
    import torch
    tensors = dict(v_out=v_out, conv_state=conv_state, x=x, weight=weight)
    if q_out is not None:
        tensors.update(q_out=q_out, k_out=k_out)
    if bias is not None:
        tensors['bias'] = bias
    _device_contiguous(**tensors)
    B, C, L = conv_state.shape
    K = weight.shape[1]
    key_dim = 0 if q_out is None else q_out.shape[1]
    value_dim = v_out.shape[1]
    dt = conv_state.dtype
    _require(dt in (torch.float32, torch.bfloat16) and all(t.dtype == dt for t in tensors.values()),
             'causal_conv1d_update: all tensors fp32 or all bf16')
    _require(2 * key_dim + value_dim == C and tuple(x.shape) == (B, C) and tuple(weight.shape) == (C, K)
             and tuple(v_out.shape) == (B, value_dim), 'causal_conv1d_update: shapes')
    _require(q_out is None or (tuple(q_out.shape) == tuple(k_out.shape) == (B, key_dim)),
             'causal_conv1d_update: q_out/k_out shape')
    _require(bias is None or tuple(bias.shape) == (C,), 'causal_conv1d_update: bias shape')
    _require(activation in (None, 'silu'), "causal_conv1d_update: activation is None or 'silu'")
    null = c_void_p(None)
    library().causal_conv1d_update_launcher(
        _ptr(q_out) if q_out is not None else null, _ptr(k_out) if q_out is not None else null, _ptr(v_out),
        _ptr(conv_state), _ptr(x), _ptr(weight), _ptr(bias) if bias is not None else null, B, key_dim,
        value_dim, L, K, 1 if activation == 'silu' else 0, 0 if dt == torch.float32 else 1, config,
        _stream(stream))
    check_status('causal_conv1d_update_launcher')
    return q_out, k_out, v_out


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


def sparse_mla_decode_static_launch(out, q, kv, idx, sm_scale=192 ** -0.5, config=0, stream=None):
    """sparse_mla_decode_launch without a workspace: the split partials go to the library's static device array
    (``sparse_mla_decode_static_scratch_bytes()``); nothing is allocated. Calls that overlap on one GPU race."""
    import torch
    _device_contiguous(out=out, q=q, kv=kv, idx=idx)
    B, H, d_qk = q.shape
    N = kv.shape[1]
    topk = idx.shape[1]
    d_v = out.shape[2]
    _require(q.dtype == kv.dtype == torch.bfloat16, 'sparse_mla: q, kv must be bf16')
    _require(out.dtype in (torch.bfloat16, torch.float32), 'sparse_mla: out must be bf16 or fp32')
    _require(idx.dtype == torch.int32, 'sparse_mla: idx must be int32')
    _require(tuple(kv.shape) == (B, N, d_qk) and tuple(idx.shape) == (B, topk), 'sparse_mla: kv/idx shape')
    _require(tuple(out.shape) == (B, H, d_v), 'sparse_mla: out shape')
    library().sparse_mla_decode_static_launcher(_ptr(out), _ptr(q), _ptr(kv), _ptr(idx), B, H, N, topk, d_qk, d_v,
                                                float(sm_scale), 0 if out.dtype == torch.bfloat16 else 1, config,
                                                _stream(stream))
    check_status('sparse_mla_decode_static_launcher')
    return out


def sparse_mla_decode_paged_launch(out, q, kv_pool, block_table, idx, workspace, sm_scale=192 ** -0.5,
                                   config=0, stream=None):
    """As ``sparse_mla_decode_launch`` over a paged cache: kv_pool [n_pages, page_size, 576] bf16,
    block_table [B, max_pages] int32 or None (idx then holds pool rows), idx [B, topk] int32."""
    import torch
    _device_contiguous(out=out, q=q, kv_pool=kv_pool, idx=idx, workspace=workspace)
    B, H, d_qk = q.shape
    n_pages, page_size = kv_pool.shape[0], kv_pool.shape[1]
    topk = idx.shape[1]
    d_v = out.shape[2]
    _require(q.dtype == kv_pool.dtype == torch.bfloat16, 'sparse_mla: q, kv_pool must be bf16')
    _require(out.dtype in (torch.bfloat16, torch.float32), 'sparse_mla: out must be bf16 or fp32')
    _require(idx.dtype == torch.int32, 'sparse_mla: idx must be int32')
    _require(tuple(kv_pool.shape) == (n_pages, page_size, d_qk) and tuple(idx.shape) == (B, topk),
             'sparse_mla: kv_pool/idx shape')
    _require(tuple(out.shape) == (B, H, d_v), 'sparse_mla: out shape')
    max_pages = 0
    if block_table is not None:
        _device_contiguous(block_table=block_table)
        _require(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] == B,
                 'sparse_mla: block_table must be int32 [B, max_pages]')
        max_pages = block_table.shape[1]
    library().sparse_mla_decode_paged_launcher(
        _ptr(out), _ptr(q), _ptr(kv_pool), _ptr(block_table) if block_table is not None else None,
        _ptr(idx), _ptr(workspace), workspace.numel() * workspace.element_size(), B, H, n_pages,
        page_size, max_pages, topk, d_qk, d_v, float(sm_scale),
        0 if out.dtype == torch.bfloat16 else 1, config, _stream(stream))
    check_status('sparse_mla_decode_paged_launcher')
    return out


LATENT_ROW_BYTES = 656


def mla_latent_quant_launch(cache, kv, config=0, stream=None):
    """cache [..., 656] uint8 <- the e4m3 storage form of the latent rows kv [..., 576] bf16 (512 codes, 4 fp32
    block scales, 64 bf16 rope values per row). config 32: power-of-two scales."""
    import torch
    _device_contiguous(cache=cache, kv=kv)
    _require(kv.dtype == torch.bfloat16 and cache.dtype == torch.uint8, 'mla_latent_quant: kv bf16, cache uint8')
    _require(kv.shape[-1] == 576 and cache.shape[-1] == LATENT_ROW_BYTES and tuple(kv.shape[:-1]) == tuple(cache.shape[:-1]),
             'mla_latent_quant: kv [..., 576], cache [..., 656]')
    rows = kv.numel() // 576
    library().mla_latent_quant_launcher(_ptr(cache), _ptr(kv), rows, config, _stream(stream))
    check_status('mla_latent_quant_launcher')
    return cache


def sparse_mla_fp8_workspace_bytes(batch, n_heads, topk, config=0):
    return int(library().sparse_mla_decode_fp8_workspace_bytes(batch, n_heads, topk, config))


def sparse_mla_decode_fp8_launch(out, q, kv_fp8, idx, workspace, sm_scale=192 ** -0.5, config=0, stream=None):
    """As ``sparse_mla_decode_launch`` over kv_fp8 [B, N, 656] uint8, the e4m3 storage form of the latent cache.
    ``workspace``: at least ``sparse_mla_fp8_workspace_bytes`` bytes."""
    import torch
    _device_contiguous(out=out, q=q, kv_fp8=kv_fp8, idx=idx, workspace=workspace)
    B, H, d_qk = q.shape
    N = kv_fp8.shape[1]
    topk = idx.shape[1]
    d_v = out.shape[2]
    _require(q.dtype == torch.bfloat16 and kv_fp8.dtype == torch.uint8, 'sparse_mla_fp8: q bf16, kv_fp8 uint8')
    _require(out.dtype in (torch.bfloat16, torch.float32), 'sparse_mla_fp8: out must be bf16 or fp32')
    _require(idx.dtype == torch.int32, 'sparse_mla_fp8: idx must be int32')
    _require(tuple(kv_fp8.shape) == (B, N, LATENT_ROW_BYTES) and tuple(idx.shape) == (B, topk),
             'sparse_mla_fp8: kv_fp8 [B, N, 656], idx [B, topk]')
    _require(tuple(out.shape) == (B, H, d_v), 'sparse_mla_fp8: out shape')
    _require(workspace.dtype == torch.uint8, 'sparse_mla_fp8: workspace must be uint8')
    library().sparse_mla_decode_fp8_launcher(
        _ptr(out), _ptr(q), _ptr(kv_fp8), _ptr(idx), _ptr(workspace), workspace.numel(), B, H, N, topk, d_qk, d_v,
        float(sm_scale), 0 if out.dtype == torch.bfloat16 else 1, config, _stream(stream))
    check_status('sparse_mla_decode_fp8_launcher')
    return out


def sparse_mla_decode_fp8_paged_launch(out, q, kv_pool_fp8, block_table, idx, workspace, sm_scale=192 ** -0.5,
                                       config=0, stream=None):
    """As ``sparse_mla_decode_paged_launch`` over kv_pool_fp8 [n_pages, page_size, 656] uint8 (the e4m3 storage
    form); ``workspace``: at least ``sparse_mla_fp8_workspace_bytes`` bytes."""
    import torch
    _device_contiguous(out=out, q=q, kv_pool_fp8=kv_pool_fp8, idx=idx, workspace=workspace)
    B, H, d_qk = q.shape
    n_pages, page_size = kv_pool_fp8.shape[0], kv_pool_fp8.shape[1]
    topk = idx.shape[1]
    d_v = out.shape[2]
    _require(q.dtype == torch.bfloat16 and kv_pool_fp8.dtype == torch.uint8, 'sparse_mla_fp8: q bf16, kv_pool_fp8 uint8')
    _require(out.dtype in (torch.bfloat16, torch.float32), 'sparse_mla_fp8: out must be bf16 or fp32')
    _require(idx.dtype == torch.int32, 'sparse_mla_fp8: idx must be int32')
    _require(tuple(kv_pool_fp8.shape) == (n_pages, page_size, LATENT_ROW_BYTES) and tuple(idx.shape) == (B, topk),
             'sparse_mla_fp8: kv_pool_fp8 [n_pages, page, 656], idx [B, topk]')
    _require(tuple(out.shape) == (B, H, d_v), 'sparse_mla_fp8: out shape')
    max_pages = 0
    if block_table is not None:
        _device_contiguous(block_table=block_table)
        _require(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] == B,
                 'sparse_mla_fp8: block_table must be int32 [B, max_pages]')
        max_pages = block_table.shape[1]
    library().sparse_mla_decode_fp8_paged_launcher(
        _ptr(out), _ptr(q), _ptr(kv_pool_fp8), _ptr(block_table) if block_table is not None else None,
        _ptr(idx), _ptr(workspace), workspace.numel() * workspace.element_size(), B, H, n_pages,
        page_size, max_pages, topk, d_qk, d_v, float(sm_scale),
        0 if out.dtype == torch.bfloat16 else 1, config, _stream(stream))
    check_status('sparse_mla_decode_fp8_paged_launcher')
    return out


def mla_index_scores_launch(scores, q, k_cache, w, lengths=None, scale=128 ** -0.5, stream=None):
    """scores [B, N] fp32 <- sum_h w[b,h] * relu(scale * q[b,h] . k_cache[b,t]); -inf at t >= lengths[b].
    q [B, Hi, 128] bf16, k_cache [B, N, 128] bf16, w [B, Hi] fp32."""
    import torch
    _device_contiguous(scores=scores, q=q, k_cache=k_cache, w=w)
    B, Hi, D = q.shape
    N = k_cache.shape[1]
    _require(q.dtype == k_cache.dtype == torch.bfloat16 and w.dtype == scores.dtype == torch.float32,
             'mla_index_scores: q, k_cache bf16; w, scores fp32')
    _require(tuple(k_cache.shape) == (B, N, D) and tuple(w.shape) == (B, Hi) and tuple(scores.shape) == (B, N),
             'mla_index_scores: shapes')
    if lengths is not None:
        _device_contiguous(lengths=lengths)
        _require(lengths.dtype == torch.int32 and tuple(lengths.shape) == (B,), 'mla_index_scores: lengths int32 [B]')
    library().mla_index_scores_launcher(_ptr(scores), _ptr(q), _ptr(k_cache), _ptr(w),
                                        _ptr(lengths) if lengths is not None else c_void_p(None), B, Hi, N, D,
                                        float(scale), 0, _stream(stream))
    check_status('mla_index_scores_launcher')
    return scores


def mla_index_scores_paged_launch(scores, q, k_pool, block_table, w, lengths=None, scale=128 ** -0.5, stream=None):
    """As ``mla_index_scores_launch`` over a paged key cache: k_pool [n_pages, page, 128] bf16, block_table
    [B, max_pages] int32; scores [B, max_pages * page] over logical positions."""
    import torch
    _device_contiguous(scores=scores, q=q, k_pool=k_pool, block_table=block_table, w=w)
    B, Hi, D = q.shape
    n_pages, page = k_pool.shape[0], k_pool.shape[1]
    max_pages = block_table.shape[1]
    _require(q.dtype == k_pool.dtype == torch.bfloat16 and w.dtype == scores.dtype == torch.float32,
             'mla_index_scores: q, k_pool bf16; w, scores fp32')
    _require(block_table.dtype == torch.int32 and block_table.shape[0] == B, 'mla_index_scores: block_table int32 [B, P]')
    _require(tuple(k_pool.shape) == (n_pages, page, D) and tuple(w.shape) == (B, Hi)
             and tuple(scores.shape) == (B, max_pages * page), 'mla_index_scores: shapes')
    if lengths is not None:
        _device_contiguous(lengths=lengths)
        _require(lengths.dtype == torch.int32 and tuple(lengths.shape) == (B,), 'mla_index_scores: lengths int32 [B]')
    library().mla_index_scores_paged_launcher(
        _ptr(scores), _ptr(q), _ptr(k_pool), _ptr(block_table), _ptr(w),
        _ptr(lengths) if lengths is not None else c_void_p(None), B, Hi, n_pages, page, max_pages, D, float(scale),
        0, _stream(stream))
    check_status('mla_index_scores_paged_launcher')
    return scores


def _is_e4m3(t):
    import torch
    return t.dtype in (torch.uint8, torch.float8_e4m3fn)


def mla_index_scores_fp8_launch(scores, q, k_cache, k_scale, w, lengths=None, scale=128 ** -0.5, stream=None):
    """scores [B, N] fp32 <- k_scale[b,t] * sum_h w[b,h] * relu(scale * q[b,h] . k_cache[b,t]); -inf at
    t >= lengths[b]. q [B, Hi, 128] and k_cache [B, N, 128] e4m3 codes (uint8 or float8_e4m3fn),
    k_scale [B, N] fp32, w [B, Hi] fp32 (head weight times the scale of that head's q)."""
    import torch
    _device_contiguous(scores=scores, q=q, k_cache=k_cache, k_scale=k_scale, w=w)
    B, Hi, D = q.shape
    N = k_cache.shape[1]
    _require(_is_e4m3(q) and _is_e4m3(k_cache) and k_scale.dtype == w.dtype == scores.dtype == torch.float32,
             'mla_index_scores_fp8: q, k_cache e4m3 codes; k_scale, w, scores fp32')
    _require(tuple(k_cache.shape) == (B, N, D) and tuple(k_scale.shape) == (B, N) and tuple(w.shape) == (B, Hi)
             and tuple(scores.shape) == (B, N), 'mla_index_scores_fp8: shapes')
    if lengths is not None:
        _device_contiguous(lengths=lengths)
        _require(lengths.dtype == torch.int32 and tuple(lengths.shape) == (B,),
                 'mla_index_scores_fp8: lengths int32 [B]')
    library().mla_index_scores_fp8_launcher(_ptr(scores), _ptr(q), _ptr(k_cache), _ptr(k_scale), _ptr(w),
                                            _ptr(lengths) if lengths is not None else c_void_p(None), B, Hi, N, D,
                                            float(scale), 0, _stream(stream))
    check_status('mla_index_scores_fp8_launcher')
    return scores


def mla_index_scores_fp8_paged_launch(scores, q, k_pool, k_scale_pool, block_table, w, lengths=None,
                                      scale=128 ** -0.5, stream=None):
    """As ``mla_index_scores_fp8_launch`` over a paged key cache: k_pool [n_pages, page, 128] e4m3 codes,
    k_scale_pool [n_pages, page] fp32, block_table [B, max_pages] int32; scores [B, max_pages * page]."""
    import torch
    _device_contiguous(scores=scores, q=q, k_pool=k_pool, k_scale_pool=k_scale_pool, block_table=block_table, w=w)
    B, Hi, D = q.shape
    n_pages, page = k_pool.shape[0], k_pool.shape[1]
    max_pages = block_table.shape[1]
    _require(_is_e4m3(q) and _is_e4m3(k_pool) and k_scale_pool.dtype == w.dtype == scores.dtype == torch.float32,
             'mla_index_scores_fp8: q, k_pool e4m3 codes; k_scale_pool, w, scores fp32')
    _require(block_table.dtype == torch.int32 and block_table.shape[0] == B,
             'mla_index_scores_fp8: block_table int32 [B, P]')
    _require(tuple(k_pool.shape) == (n_pages, page, D) and tuple(k_scale_pool.shape) == (n_pages, page)
             and tuple(w.shape) == (B, Hi) and tuple(scores.shape) == (B, max_pages * page),
             'mla_index_scores_fp8: shapes')
    if lengths is not None:
        _device_contiguous(lengths=lengths)
        _require(lengths.dtype == torch.int32 and tuple(lengths.shape) == (B,),
                 'mla_index_scores_fp8: lengths int32 [B]')
    library().mla_index_scores_fp8_paged_launcher(
        _ptr(scores), _ptr(q), _ptr(k_pool), _ptr(k_scale_pool), _ptr(block_table), _ptr(w),
        _ptr(lengths) if lengths is not None else c_void_p(None), B, Hi, n_pages, page, max_pages, D, float(scale),
        0, _stream(stream))
    check_status('mla_index_scores_fp8_paged_launcher')
    return scores


def topk_select_launch(idx_out, scores, lengths=None, stream=None):
    """idx_out [B, k] int32 <- indices of the k largest of scores [B, n] fp32 per row (first lengths[b]
    entries only, if given), ties to the lower index, ascending index order, -1 padding."""
    import torch
    _device_contiguous(idx_out=idx_out, scores=scores)
    B, n = scores.shape
    _require(scores.dtype == torch.float32 and idx_out.dtype == torch.int32, 'topk_select: scores fp32, idx int32')
    _require(idx_out.dim() == 2 and idx_out.shape[0] == B, 'topk_select: idx_out [B, k]')
    if lengths is not None:
        _device_contiguous(lengths=lengths)
        _require(lengths.dtype == torch.int32 and tuple(lengths.shape) == (B,), 'topk_select: lengths int32 [B]')
    library().topk_select_launcher(_ptr(idx_out), _ptr(scores),
                                   _ptr(lengths) if lengths is not None else c_void_p(None), B, n,
                                   idx_out.shape[1], 0, _stream(stream))
    check_status('topk_select_launcher')
    return idx_out


MOE_WORKSPACE_FIELDS = ('ids', 'weights', 'expert_offsets', 'sorted_pairs', 'pair_pos', 'x_q', 'x_s',
                        'h_q', 'h_s', 'y', 'y_scale')


def moe_workspace_bytes(tokens, hidden, inter, n_experts, top_k=8):
    return int(library().moe_fp8_workspace_bytes(tokens, hidden, inter, n_experts, top_k))


def moe_workspace_views(workspace, tokens, hidden, inter, n_experts, top_k=8):
    """Typed views of the intermediate buffers inside a workspace tensor (uint8, 1-D). ``y`` is laid out as
    fp32 rows; when the layer ran the LDS-tiled GEMMs (``moe_fp8_uses_tiled_gemms`` returns 1) it holds fp16 rows
    with the scales in ``y_scale`` instead and must be read through ``moe_expert_outputs``."""
    import torch
    offs = (c_size_t * len(MOE_WORKSPACE_FIELDS))()
    n = library().moe_fp8_workspace_layout(offs, len(MOE_WORKSPACE_FIELDS), tokens, hidden, inter, n_experts, top_k)
    _require(n == len(MOE_WORKSPACE_FIELDS), f'moe_fp8_workspace_layout has {n} fields, this module knows '
                                             f'{len(MOE_WORKSPACE_FIELDS)}')
    pairs = tokens * top_k
    spec = {
        'ids': (torch.int32, (tokens, top_k)), 'weights': (torch.float32, (tokens, top_k)),
        'expert_offsets': (torch.int32, (n_experts + 1,)), 'sorted_pairs': (torch.int32, (pairs,)),
        'pair_pos': (torch.int32, (pairs,)), 'x_q': (torch.float8_e4m3fn, (tokens, hidden)),
        'x_s': (torch.float32, (tokens, hidden // 128)), 'h_q': (torch.float8_e4m3fn, (pairs, inter)),
        'h_s': (torch.float32, (pairs, inter // 128)), 'y': (torch.float32, (pairs, hidden)),
        'y_scale': (torch.float32, (pairs, (hidden + 255) // 256)),
    }
    views = {}
    for name, off in zip(MOE_WORKSPACE_FIELDS, offs):
        dtype, shape = spec[name]
        n = 1
        for d in shape:
            n *= d
        nbytes = n * torch.empty((), dtype=dtype).element_size()
        views[name] = workspace[off:off + nbytes].view(dtype).view(shape)
    return views


def moe_expert_outputs(views, tokens, hidden, inter, n_experts, top_k=8, config=0):
    """The expert outputs y [tokens*top_k, hidden] of a finished layer as fp32, whichever way the layer stored
    them: fp32 rows (weight-streaming GEMMs) or fp16 rows with power-of-two scales (LDS-tiled GEMMs)."""
    import torch
    tiled = library().moe_fp8_uses_tiled_gemms(tokens, hidden, inter, n_experts, top_k, config)
    _require(tiled >= 0, 'moe_expert_outputs: unsupported shape')
    if not tiled:
        return views['y']
    pairs = tokens * top_k
    half = views['y'].reshape(-1).view(torch.float16)[:pairs * hidden].view(pairs, hidden)
    return half.float() * views['y_scale'].repeat_interleave(256, dim=1)


def moe_route_launch(ids, weights, logits, stream=None):
    import torch
    _device_contiguous(ids=ids, weights=weights, logits=logits)
    T, E = logits.shape
    k = ids.shape[1]
    _require(logits.dtype == torch.float32 and weights.dtype == torch.float32 and ids.dtype == torch.int32,
             'moe_route: dtypes')
    _require(tuple(ids.shape) == (T, k) and tuple(weights.shape) == (T, k), 'moe_route: shapes')
    library().moe_route_launcher(_ptr(ids), _ptr(weights), _ptr(logits), T, E, k, 0, _stream(stream))
    check_status('moe_route_launcher')
    return ids, weights


def moe_router_logits_workspace_bytes(tokens, hidden, n_experts):
    return int(library().moe_router_logits_workspace_bytes(tokens, hidden, n_experts))


def moe_router_logits_launch(logits, x, w, workspace=None, stream=None):
    """logits [T, E] fp32 <- x [T, H] (bf16 or fp32) @ w [E, H]^T (fp32); ``workspace``: uint8 device tensor of
    ``moe_router_logits_workspace_bytes`` bytes (None when that is 0)."""
    import torch
    _device_contiguous(logits=logits, x=x, w=w)
    T, H = x.shape
    E = w.shape[0]
    _require(x.dtype in (torch.float32, torch.bfloat16) and w.dtype == logits.dtype == torch.float32,
             'moe_router_logits: x fp32 or bf16, w and logits fp32')
    _require(tuple(w.shape) == (E, H) and tuple(logits.shape) == (T, E), 'moe_router_logits: shapes')
    ws_ptr, ws_bytes = c_void_p(None), 0
    if workspace is not None:
        _device_contiguous(workspace=workspace)
        ws_ptr, ws_bytes = _ptr(workspace), workspace.numel() * workspace.element_size()
    library().moe_router_logits_launcher(_ptr(logits), _ptr(x), _ptr(w), ws_ptr, ws_bytes, T, H, E,
                                         0 if x.dtype == torch.float32 else 1, 0, _stream(stream))
    check_status('moe_router_logits_launcher')
    return logits


def moe_router_split_weight_launch(planes, w, stream=None):
    """planes [3, E, H] bf16 <- the three bf16 numbers whose sum is w [E, H] fp32 (done once per weight)."""
    import torch
    _device_contiguous(planes=planes, w=w)
    E, H = w.shape
    _require(w.dtype == torch.float32 and planes.dtype == torch.bfloat16 and tuple(planes.shape) == (3, E, H),
             'moe_router_split_weight: w fp32 [E, H], planes bf16 [3, E, H]')
    library().moe_router_split_weight_launcher(_ptr(planes), _ptr(w), E, H, _stream(stream))
    check_status('moe_router_split_weight_launcher')
    return planes


def moe_router_logits_split_launch(logits, x, planes, workspace=None, stream=None):
    """``moe_router_logits_launch`` for a bf16 x and the weight given as its three bf16 planes [3, E, H]."""
    import torch
    _device_contiguous(logits=logits, x=x, planes=planes)
    T, H = x.shape
    E = planes.shape[1]
    _require(x.dtype == planes.dtype == torch.bfloat16 and logits.dtype == torch.float32,
             'moe_router_logits_split: x and planes bf16, logits fp32')
    _require(tuple(planes.shape) == (3, E, H) and tuple(logits.shape) == (T, E), 'moe_router_logits_split: shapes')
    ws_ptr, ws_bytes = c_void_p(None), 0
    if workspace is not None:
        _device_contiguous(workspace=workspace)
        ws_ptr, ws_bytes = _ptr(workspace), workspace.numel() * workspace.element_size()
    library().moe_router_logits_split_launcher(_ptr(logits), _ptr(x), _ptr(planes), ws_ptr, ws_bytes, T, H, E, 0,
                                               _stream(stream))
    check_status('moe_router_logits_split_launcher')
    return logits


def moe_route_grouped_launch(ids, weights, logits, bias, n_group, topk_group, normalise=True,
                             routed_scaling_factor=1.0, stream=None):
    """ids/weights [T, top_k] <- group-limited, bias-corrected top-k of logits [T, E] (bias [E] or None)."""
    import torch
    _device_contiguous(ids=ids, weights=weights, logits=logits)
    T, E = logits.shape
    top_k = ids.shape[1]
    _require(ids.dtype == torch.int32 and weights.dtype == logits.dtype == torch.float32,
             'moe_route_grouped: ids int32, weights/logits fp32')
    _require(tuple(ids.shape) == tuple(weights.shape) == (T, top_k), 'moe_route_grouped: ids/weights shape')
    if bias is not None:
        _device_contiguous(bias=bias)
        _require(bias.dtype == torch.float32 and tuple(bias.shape) == (E,), 'moe_route_grouped: bias fp32 [E]')
    library().moe_route_grouped_launcher(_ptr(ids), _ptr(weights), _ptr(logits),
                                         _ptr(bias) if bias is not None else c_void_p(None), T, E, top_k,
                                         n_group, topk_group, 1 if normalise else 0,
                                         float(routed_scaling_factor), 0, _stream(stream))
    check_status('moe_route_grouped_launcher')
    return ids, weights


def moe_sort_launch(ids, n_experts, stream=None):
    """Returns (sorted_pairs, pair_pos, expert_offsets) int32 device tensors."""
    import torch
    _device_contiguous(ids=ids)
    _require(ids.dtype == torch.int32 and ids.dim() == 2, 'moe_sort: ids must be int32 [T, k]')
    T, k = ids.shape
    dev = ids.device
    sorted_pairs = torch.empty(T * k, dtype=torch.int32, device=dev)
    pair_pos = torch.empty(T * k, dtype=torch.int32, device=dev)
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    scratch = torch.empty(((T + 255) // 256) * n_experts, dtype=torch.int32, device=dev)
    library().moe_sort_launcher(_ptr(sorted_pairs), _ptr(pair_pos), _ptr(offsets), _ptr(scratch),
                                _ptr(ids), T, n_experts, k, 0, _stream(stream))
    check_status('moe_sort_launcher')
    return sorted_pairs, pair_pos, offsets


CONFIG_UE8M0 = 32   # config bit of the MoE launchers: power-of-two block scales


def moe_quant_bf16_launch(q, scales, x, stream=None, config=0):
    import torch
    _device_contiguous(q=q, scales=scales, x=x)
    R, C = x.shape
    _require(x.dtype == torch.bfloat16 and scales.dtype == torch.float32, 'moe_quant: dtypes')
    _require(q.element_size() == 1 and tuple(q.shape) == (R, C), 'moe_quant: q must be 1-byte [R, C]')
    _require(tuple(scales.shape) == (R, C // 128), 'moe_quant: scales shape')
    library().moe_quant_bf16_launcher(_ptr(q), _ptr(scales), _ptr(x), R, C, config, _stream(stream))
    check_status('moe_quant_bf16_launcher')
    return q, scales


def moe_rmsnorm_quant_launch(q, scales, y, x, weight, eps=1e-6, config=0, stream=None):
    """y (bf16 or None) = RMS norm of x [R, C] bf16 with weight [C] bf16; q, scales = its activation quantisation."""
    import torch
    _device_contiguous(q=q, scales=scales, x=x, weight=weight)
    R, C = x.shape
    _require(x.dtype == weight.dtype == torch.bfloat16 and scales.dtype == torch.float32, 'moe_rmsnorm_quant: dtypes')
    _require(q.element_size() == 1 and tuple(q.shape) == (R, C) and tuple(scales.shape) == (R, C // 128)
             and tuple(weight.shape) == (C,), 'moe_rmsnorm_quant: shapes')
    if y is not None:
        _device_contiguous(y=y)
        _require(y.dtype == torch.bfloat16 and tuple(y.shape) == (R, C), 'moe_rmsnorm_quant: y bf16 [R, C]')
    library().moe_rmsnorm_quant_launcher(_ptr(q), _ptr(scales), _ptr(y) if y is not None else c_void_p(None),
                                         _ptr(x), _ptr(weight), float(eps), R, C, config, _stream(stream))
    check_status('moe_rmsnorm_quant_launcher')
    return q, scales, y


def moe_fp8_launch(out, x, logits, w13_q, w13_s, w2_q, w2_s, workspace, top_k=8, config=0, stream=None):
    """The whole layer; ``out`` [T, H] bf16 (or fp32 for the unrounded values)."""
    import torch
    _device_contiguous(out=out, x=x, logits=logits, w13_q=w13_q, w13_s=w13_s, w2_q=w2_q, w2_s=w2_s,
                       workspace=workspace)
    T, H = x.shape
    E, I2, _ = w13_q.shape
    I = I2 // 2
    _require(x.dtype == torch.bfloat16 and logits.dtype == torch.float32, 'moe_fp8: x bf16, logits fp32')
    _require(out.dtype in (torch.bfloat16, torch.float32) and tuple(out.shape) == (T, H), 'moe_fp8: out')
    _require(w13_q.element_size() == 1 and w2_q.element_size() == 1, 'moe_fp8: weights must be e4m3')
    _require(tuple(w13_q.shape) == (E, 2 * I, H) and tuple(w2_q.shape) == (E, H, I), 'moe_fp8: weight shapes')
    _require(tuple(w13_s.shape) == (E, 2 * I // 128, H // 128) and tuple(w2_s.shape) == (E, H // 128, I // 128),
             'moe_fp8: scale shapes')
    _require(w13_s.dtype == torch.float32 and w2_s.dtype == torch.float32, 'moe_fp8: scales fp32')
    _require(tuple(logits.shape) == (T, E), 'moe_fp8: logits shape')
    library().moe_fp8_launcher(_ptr(out), _ptr(x), _ptr(logits), _ptr(w13_q), _ptr(w13_s), _ptr(w2_q),
                               _ptr(w2_s), _ptr(workspace), workspace.numel() * workspace.element_size(),
                               T, H, I, E, top_k, 0 if out.dtype == torch.bfloat16 else 1, config,
                               _stream(stream))
    check_status('moe_fp8_launcher')
    return out


def moe_shared_workspace_bytes(tokens, hidden, inter, shared_inter, n_experts, top_k=8):
    return int(library().moe_fp8_shared_workspace_bytes(tokens, hidden, inter, shared_inter, n_experts, top_k))


def moe_fp8_shared_launch(out, x, logits, w13_q, w13_s, w2_q, w2_s, sw13_q, sw13_s, sw2_q, sw2_s, workspace,
                          top_k=8, config=0, stream=None):
    """The layer plus a shared expert (sw13_q [2*Is, H], sw13_s [2*Is/128, H/128], sw2_q [H, Is],
    sw2_s [H/128, Is/128]) applied to every token with weight 1."""
    import torch
    _device_contiguous(out=out, x=x, logits=logits, w13_q=w13_q, w13_s=w13_s, w2_q=w2_q, w2_s=w2_s,
                       sw13_q=sw13_q, sw13_s=sw13_s, sw2_q=sw2_q, sw2_s=sw2_s, workspace=workspace)
    T, H = x.shape
    E, I2, _ = w13_q.shape
    I = I2 // 2
    Is = sw13_q.shape[0] // 2
    _require(x.dtype == torch.bfloat16 and logits.dtype == torch.float32, 'moe_fp8: x bf16, logits fp32')
    _require(out.dtype in (torch.bfloat16, torch.float32) and tuple(out.shape) == (T, H), 'moe_fp8: out')
    _require(all(t.element_size() == 1 for t in (w13_q, w2_q, sw13_q, sw2_q)), 'moe_fp8: weights must be e4m3')
    _require(tuple(w13_q.shape) == (E, 2 * I, H) and tuple(w2_q.shape) == (E, H, I), 'moe_fp8: weight shapes')
    _require(tuple(w13_s.shape) == (E, 2 * I // 128, H // 128) and tuple(w2_s.shape) == (E, H // 128, I // 128),
             'moe_fp8: scale shapes')
    _require(tuple(sw13_q.shape) == (2 * Is, H) and tuple(sw2_q.shape) == (H, Is), 'moe_fp8: shared weight shapes')
    _require(tuple(sw13_s.shape) == (2 * Is // 128, H // 128) and tuple(sw2_s.shape) == (H // 128, Is // 128),
             'moe_fp8: shared scale shapes')
    _require(all(t.dtype == torch.float32 for t in (w13_s, w2_s, sw13_s, sw2_s)), 'moe_fp8: scales fp32')
    _require(tuple(logits.shape) == (T, E), 'moe_fp8: logits shape')
    library().moe_fp8_shared_launcher(
        _ptr(out), _ptr(x), _ptr(logits), _ptr(w13_q), _ptr(w13_s), _ptr(w2_q), _ptr(w2_s), _ptr(sw13_q),
        _ptr(sw13_s), _ptr(sw2_q), _ptr(sw2_s), _ptr(workspace), workspace.numel() * workspace.element_size(),
        T, H, I, Is, E, top_k, 0 if out.dtype == torch.bfloat16 else 1, config, _stream(stream))
    check_status('moe_fp8_shared_launcher')
    return out


def moe_fp8_fused_shared_launch(out, x, logits, w13_q, w13_s, w2_q, w2_s, workspace, top_k=8, config=0,
                                stream=None):
    """The layer with the shared expert stored as the last of E+1 experts in the weight tensors; logits [T, E].
    ``workspace``: ``moe_workspace_bytes(T, H, I, E + 1, top_k + 1)`` bytes."""
    import torch
    _device_contiguous(out=out, x=x, logits=logits, w13_q=w13_q, w13_s=w13_s, w2_q=w2_q, w2_s=w2_s,
                       workspace=workspace)
    T, H = x.shape
    E1, I2, _ = w13_q.shape
    I, E = I2 // 2, E1 - 1
    _require(x.dtype == torch.bfloat16 and logits.dtype == torch.float32, 'moe_fp8: x bf16, logits fp32')
    _require(out.dtype in (torch.bfloat16, torch.float32) and tuple(out.shape) == (T, H), 'moe_fp8: out')
    _require(w13_q.element_size() == 1 and w2_q.element_size() == 1, 'moe_fp8: weights must be e4m3')
    _require(tuple(w13_q.shape) == (E1, 2 * I, H) and tuple(w2_q.shape) == (E1, H, I), 'moe_fp8: weight shapes')
    _require(tuple(w13_s.shape) == (E1, 2 * I // 128, H // 128) and tuple(w2_s.shape) == (E1, H // 128, I // 128),
             'moe_fp8: scale shapes')
    _require(w13_s.dtype == torch.float32 and w2_s.dtype == torch.float32, 'moe_fp8: scales fp32')
    _require(tuple(logits.shape) == (T, E), 'moe_fp8: logits [T, E] for E + 1 stored experts')
    library().moe_fp8_fused_shared_launcher(
        _ptr(out), _ptr(x), _ptr(logits), _ptr(w13_q), _ptr(w13_s), _ptr(w2_q), _ptr(w2_s), _ptr(workspace),
        workspace.numel() * workspace.element_size(), T, H, I, E, top_k,
        0 if out.dtype == torch.bfloat16 else 1, config, _stream(stream))
    check_status('moe_fp8_fused_shared_launcher')
    return out

