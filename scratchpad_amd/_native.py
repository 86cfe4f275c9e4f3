"""ctypes binding of ``libscratchpad_hip.so`` (C ABI: ``include/scratchpad_hip.h``).

There is no fallback: if the library is missing or a call fails, a ``RuntimeError`` is raised
(the reference's convention - exceptions in the forward thread are logged and the parent is
signalled, managers/tp_worker_client.py:110-116).  Tensors are passed as raw device pointers on
``torch.cuda.current_stream()``; nothing here synchronises.
"""
import ctypes
import os
import weakref
from typing import Optional, Tuple

import torch

# SP_NATIVE_LIB names a diagnostic build under lib/ (A/B runs of a kernel variant through the whole model); unset = the product
_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib",
                         os.environ.get("SP_NATIVE_LIB") or "libscratchpad_hip.so")
_lib = None

SP_F32, SP_F16, SP_BF16 = 0, 1, 2
_DTYPES = {torch.float32: SP_F32, torch.float16: SP_F16, torch.bfloat16: SP_BF16}
SP_FP8_E5M2 = 3
SP_OK, SP_ERR_INVALID_ARG, SP_ERR_UNSUPPORTED, SP_ERR_WORKSPACE, SP_ERR_LAUNCH = 0, -1, -2, -3, -4     # sp_status
_FP8_POOL_DTYPES = (torch.uint8, torch.float8_e5m2)


def _kv_layout(k_buffer: torch.Tensor, v_buffer: torch.Tensor, what: str, same_stride: bool = True) -> None:
    """The pool views every kernel assumes: [P+1, Hkv, D] with the heads of a token contiguous (stride(1) == D,
    stride(2) == 1) and - where the ABI carries ONE token stride for both sides - the same token stride on K and V.
    MHATokenToKVPool's views satisfy this under either arena layout; anything else would gather garbage silently."""
    for name, b in (("k_buffer", k_buffer), ("v_buffer", v_buffer)):
        if b.dim() != 3 or b.stride(2) != 1 or b.stride(1) != b.shape[2] or b.stride(0) < b.shape[1] * b.shape[2]:
            raise RuntimeError(f"{what}: {name} must be [tokens, Hkv, D] with contiguous heads per token, got shape "
                               f"{tuple(b.shape)} strides {tuple(b.stride())}")
    if k_buffer.shape[:2] != v_buffer.shape[:2]:
        raise RuntimeError(f"{what}: K and V pools disagree: {tuple(k_buffer.shape)} vs {tuple(v_buffer.shape)}")
    if same_stride and v_buffer.stride(0) != k_buffer.stride(0):
        raise RuntimeError(f"{what}: K and V pools need the same token stride ({k_buffer.stride(0)} vs {v_buffer.stride(0)})")


def _kv_dt(buf: torch.Tensor, q: torch.Tensor, what: str) -> int:
    """dtype code of a KV pool buffer next to 16/32-bit q: the same type, or an e5m2 byte pool."""
    if buf.dtype == q.dtype:
        return _DTYPES[q.dtype]
    if buf.dtype in _FP8_POOL_DTYPES and q.dtype in (torch.float16, torch.bfloat16):
        return SP_FP8_E5M2
    raise RuntimeError(f"{what}: KV pool dtype {buf.dtype} does not go with q dtype {q.dtype}")


_vp, _i64, _i32, _f32, _sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float,
                              ctypes.c_size_t)

_SEQ = [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32]
# name -> (restype, argtypes); must list every symbol include/scratchpad_hip.h declares
SIGNATURES = {
    "sp_abi_version": (_i32, []),
    "sp_status_string": (ctypes.c_char_p, [_i32]),
    "sp_debug_set": (_i32, [ctypes.c_char_p, _i32]),
    "sp_debug_get": (_i32, [ctypes.c_char_p]),
    "sp_rmsnorm": (_i32, [_vp, _vp, _vp, _i64, _i32, _i64, _i64, _f32, _i32, _vp]),
    "sp_fused_add_rmsnorm": (_i32, [_vp, _vp, _vp, _i64, _i32, _i64, _i64, _f32, _i32, _vp]),
    "sp_silu_and_mul": (_i32, [_vp, _vp, _i64, _i32, _i64, _i64, _i32, _vp]),
    "sp_rotary_embedding": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i64, _i64,
                                   _i32, _vp, _i64, _vp, _vp, _vp, _i64, _i32, _vp]),
    "sp_kv_store": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i64, _i64, _i64,
                           _i64, _i32, _vp]),
    "sp_write_req_to_token": (_i32, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _i32, _vp]),
    "sp_compute_position": (_i32, [_vp, _vp, _vp, _vp, _i32, _vp]),
    "sp_clamp_position": (_i32, [_vp, _vp, _i32, _i32, _vp]),
    "sp_decode_plan_slots": (_i64, [_i32, _i64, _i64, _i32]),
    "sp_decode_attention_workspace_bytes": (_sz, [_i64, _i32, _i32]),
    "sp_decode_ranges": (_i32, [_i32, _i32, _i32, _i32, _i32]),
    "sp_decode_plan_bytes": (_sz, [_i32, _i64, _i32]),
    "sp_decode_plan": (_i32, [_vp, _sz, _vp, _i32, _i32, _i64, _i32, _i64, _i32, _vp]),
    "sp_decode_attention": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i32, _i32,
                                   _i32, _i32, _i32, _i64, _i64, _i64, _f32, _f32, _f32, _f32, _i64, _i32, _i64,
                                   _i32, _vp, _sz, _vp, _sz, _i32, _i32, _vp]),
    "sp_extend_attention_workspace_bytes": (_sz, [_i64, _i32, _i32, _i32, _i32]),
    "sp_extend_attention": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i32, _vp, _vp,
                                   _i32, _i64, _i32, _i32, _i32, _i64, _i64, _i64, _f32, _f32, _f32, _f32,
                                   _i32, _i32, _i32, _i64, _vp, _sz, _vp, _sz, _i32, _i32, _vp]),
    "sp_extend_plan_bytes": (_sz, [_i64, _i32, _i32, _i32]),
    "sp_extend_plan": (_i32, [_vp, _sz, _vp, _vp, _i32, _i32, _i64, _i32, _i32, _i32, _vp]),
    "sp_kv_store_fp8": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i64, _i64, _i64, _i64, _f32, _f32,
                               _i32, _vp]),
    "sp_argmax": (_i32, [_vp, _i64, _i32, _i32, _vp, _i32, _vp]),
    "sp_argmax_shard": (_i32, [_vp, _i64, _i32, _i32, _i32, _vp, _i32, _vp]),
    "sp_argmax_merge": (_i32, [_vp, _i32, _i32, _vp, _vp]),
    "sp_softmax_temperature": (_i32, [_vp, _i64, _vp, _i32, _i32, _vp]),
    "sp_top_k_top_p_min_p_sample": (_i32, [_vp, _i64, _vp, _vp, _vp, _vp, _i32, _i32, _vp, _vp, _vp]),
    "sp_top_k_top_p_min_p_renorm": (_i32, [_vp, _i64, _vp, _vp, _vp, _i32, _i32, _vp, _i64, _vp, _vp]),
    "sp_ar_flag_bytes": (_sz, []),
    "sp_ar_alloc": (_i32, [_vp, _sz]),
    "sp_ar_free": (_i32, [_vp]),
    "sp_ar_ipc_export": (_i32, [_vp, _vp]),
    "sp_ar_ipc_import": (_i32, [_vp, _vp]),
    "sp_ar_ipc_close": (_i32, [_vp]),
    "sp_ar_status": (_i32, [_vp, _vp]),
    "sp_ar_host_status_alloc": (_i32, [_vp, _vp]),
    "sp_ar_host_status_free": (_i32, [_vp]),
    "sp_custom_all_reduce": (_i32, [_vp, _vp, _i64, _i32, _vp, _i32, _i32, _sz, _i64, _vp, _vp]),
    "sp_fused_allreduce_add_rmsnorm": (_i32, [_vp, _vp, _vp, _i64, _i32, _i64, _i64, _f32, _i32, _vp, _i32, _i32,
                                              _sz, _i64, _vp, _vp]),
    "sp_gemm_skinny": (_i32, [_vp, _vp, _vp, _i32, _i32, _i32, _i64, _i64, _i64, _i32, _i32, _vp]),
    # ---- ABI 10 (_SEQ: the header's SP_SEQ_PARAMS)
    "sp_bigram_rows": (_i32, [_vp, _vp, _vp, _i64, *_SEQ, _i64, _i64, _i64, _vp]),
    "sp_save_last_token": (_i32, [_vp, _vp, *_SEQ, _vp]),
    "sp_save_last_rows": (_i32, [_vp, _i64, _vp, _i64, _i32, *_SEQ, _vp]),
    "sp_embed_bigram_norm": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i64, _i64, _f32, _i32, _vp]),
    "sp_add_scalar_norm": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _i64, _i64, _i64, _f32, _i32, _vp]),
    "sp_scalar_norm": (_i32, [_vp, _vp, _vp, _i64, _i32, _i64, _i64, _f32, _i32, _vp]),
    "sp_polynorm": (_i32, [_vp, _vp, _vp, _i64, _i32, _i64, _i64, _f32, _i32, _vp]),
    "sp_gate_heads": (_i32, [_vp, _vp, _vp, _i64, _i32, _i32, _i64, _i32, _vp]),
    "sp_token_shift": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _i64, *_SEQ, _i32, _vp]),
    "sp_wkv_decay": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _i32, _i64, _i32, _vp]),
    "sp_wkv_recurrence": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i64, _i64, _i64, _i64,
                                 _i64, _f32, *_SEQ, _i32, _vp]),
    "sp_rotary_interleaved": (_i32, [_vp, _vp, _vp, _f32, _i64, _i32, _i32, _i64, _i64, _i32, _i32, _vp]),
    "sp_latent_kv_store": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _f32, _vp, _i64, _i32, _i32, _i32, _f32, _i32, _vp]),
    "sp_latent_attention": (_i32, [_vp, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _i32, _i32, _i32, _i64, _i64, _f32, *_SEQ,
                                   _i32, _vp]),
    "sp_moe_route": (_i32, [_vp, _vp, _vp, _i64, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    "sp_moe_align": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _vp]),
    "sp_moe_grouped_gemm": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i64, _i64, _i32, _vp]),
    "sp_moe_glu": (_i32, [_vp, _vp, _i64, _i32, _f32, _f32, _i32, _vp]),
    "sp_moe_combine": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _i32, _i64, _i32, _vp]),
    # ---- ABI 11
    "sp_moe_softmax_topk": (_i32, [_vp, _vp, _vp, _i64, _i32, _i32, _f32, _i32, _vp]),
    "sp_embed_scale": (_i32, [_vp, _i64, _vp, _vp, _i64, _i32, _i64, _f32, _i32, _vp]),
    "sp_norm_shift": (_i32, [_vp, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i32, _f32, *_SEQ, _i32, _vp]),
    "sp_norm_save_last": (_i32, [_vp, _i64, _vp, _i64, _vp, _i32, _f32, *_SEQ, _vp]),
    "sp_stream_add": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i64, _i32, _i32, _vp]),
    "sp_qkv_rotary_store": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _f32, _vp, _vp, _vp,
                                   _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp, _f32, _i32, _vp, _i64, _vp,
                                   _i32, _vp]),
    "sp_pool_blocks": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _i32, _i32, _i32, *_SEQ, _i32, _vp]),
    "sp_window_attention": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _i32, _i32, _i32,
                                   _i32, _i64, _i32, _f32, _vp, _f32, _i32, _vp, _vp, _i64, _i32, *_SEQ, _i32, _vp]),
    "sp_small_linear_f32": (_i32, [_vp, _vp, _i64, _vp, _vp, _i64, _i32, _i32, _i32, _vp]),
    "sp_causal_conv_silu": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i32, _i32, *_SEQ, _i32, _vp]),
    "sp_mamba2_scan": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, *_SEQ, _i32, _vp]),
    "sp_gated_group_norm": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i32, _i32, _f32, _i32, _vp]),
    "sp_mlstm_scan": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp,
                             _i64, _i32, _i32, _i32, _f32, _f32, *_SEQ, _i32, _vp]),
    # ---- ABI 12
    "sp_gated_add_norm": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _vp,
                                 _i64, _i32, _f32, _i32, _vp]),
    "sp_relu_square": (_i32, [_vp, _vp, _i64, _i32, _i64, _i64, _i32, _vp]),
    "sp_scale_softcap": (_i32, [_vp, _i64, _vp, _i64, _i64, _i32, _f32, _f32, _i32, _vp]),
    "sp_delta_gates": (_i32, [_vp, _vp, _vp, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _i32, _i32, _f32, _i32, _vp]),
    "sp_delta_recurrence": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i32, _i32,
                                   _f32, *_SEQ, _i32, _vp]),
    "sp_hgrn2_scan": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _f32,
                             *_SEQ, _i32, _vp]),
    # ---- ABI 13
    "sp_add_group_norm": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _i64, _vp, _i64, _i32, _i32, _f32, _i32, _vp]),
    "sp_lowrank_gate": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _vp]),
    "sp_gated_delta_scan": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i32, _i32,
                                   _i32, _i32, _f32, *_SEQ, _i32, _vp]),
}


def _not_built(name: str):
    def missing(*_a, **_k):
        raise RuntimeError(f"{name} is not in this build of {_LIB_PATH} (it was made of the sources of one model family): "
                           "run `python -m scratchpad_amd.build` for the whole library")
    return missing


def lib_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load the HIP library (once).  Raises RuntimeError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"{_LIB_PATH} is missing: build it with `python -m scratchpad_amd.build` "
            "(or __graft_entry__.build()); there is no fallback path")
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            # a library built from the sources of one model family (build.build_native(only=...)): the rest raises on use
            setattr(lib, name, _not_built(name))
            continue
        fn.restype = res
        fn.argtypes = args
    if lib.sp_abi_version() != 13:
        raise RuntimeError("libscratchpad_hip.so ABI version mismatch")
    _lib = lib
    return lib


def _check(status: int, what: str):
    if status != 0:
        msg = load().sp_status_string(status).decode()
        raise RuntimeError(f"{what} failed: {msg} ({status})")


def debug_set(key: str, value: int) -> None:
    """Test / tuning switch of the library (sp_debug_set): "decode_kernel", "extend_defer_x10", "extend_dma" (0 = register-staged tiles),
    "extend_w64" (0 never / 1 where it pays (default) / 2 wherever it applies: the 4-wave x 64-row extend kernel),
    "extend_w64_persist" (the same three values for its persistent form on launches with a plan)."""
    _check(load().sp_debug_set(key.encode(), int(value)), f"sp_debug_set({key})")


EXTEND_KERNELS = {0: "none", 1: "extend_mfma_kernel (8 waves)", 2: "extend_w64_kernel (4 waves x 64 rows)",
                  3: "extend_w64p_kernel (persistent 4 waves x 64 rows)", 4: "row streams on the decode kernel"}


def debug_get(key: str) -> int:
    """sp_debug_get: "w64_descriptor_patched" (1 = the 4-wave x 64-row extend kernels may launch),
    "extend_last_kernel" (a key of EXTEND_KERNELS: what the last extend_attention call launched)."""
    v = int(load().sp_debug_get(key.encode()))
    if v < 0:
        raise RuntimeError(f"sp_debug_get({key}): unknown key")
    return v


def _dt(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError(f"unsupported dtype {t.dtype}") from None


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("scratchpad_amd HIP ops need device tensors (no CPU fallback)")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _rows(t: torch.Tensor) -> torch.Tensor:
    """View as [rows, inner] with a contiguous inner dimension (copy only if unavoidable)."""
    if t.dim() == 1:
        t = t.unsqueeze(0)
    if t.stride(-1) != 1:
        t = t.contiguous()
    if t.dim() > 2:
        t = t.reshape(-1, t.shape[-1])
    return t


# --------------------------------------------------------------------------- elementwise
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    _gpu(x, weight)
    x2 = _rows(x)
    out = empty_rows(x2.shape[0], x2.shape[1], x.dtype, x.device)      # spare rows behind it: see library_rows
    w = weight if weight.dtype == x.dtype else weight.to(x.dtype)
    _check(load().sp_rmsnorm(out.data_ptr(), x2.data_ptr(), w.data_ptr(), x2.shape[0], x2.shape[1],
                             x2.stride(0), out.stride(0), eps, _dt(x), _stream()), "sp_rmsnorm")
    return out.view(x.shape)


def fused_add_rmsnorm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float):
    """In place on both x and residual (flashinfer.norm.fused_add_rmsnorm contract)."""
    _gpu(x, residual, weight)
    if x.stride(-1) != 1 or residual.stride(-1) != 1 or x.dim() != 2 or residual.dim() != 2:
        raise RuntimeError("fused_add_rmsnorm needs 2-D row-contiguous x and residual (in-place op)")
    w = weight if weight.dtype == x.dtype else weight.to(x.dtype)
    _check(load().sp_fused_add_rmsnorm(x.data_ptr(), residual.data_ptr(), w.data_ptr(), x.shape[0],
                                       x.shape[1], x.stride(0), residual.stride(0), eps, _dt(x),
                                       _stream()), "sp_fused_add_rmsnorm")


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    _gpu(x)
    x2 = _rows(x)
    d = x2.shape[1] // 2
    out = empty_rows(x2.shape[0], d, x.dtype, x.device)      # spare rows behind it: see library_rows
    _check(load().sp_silu_and_mul(out.data_ptr(), x2.data_ptr(), x2.shape[0], d, x2.stride(0),
                                  out.stride(0), _dt(x), _stream()), "sp_silu_and_mul")
    return out.view(*x.shape[:-1], d)


def rotary_embedding(positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                     head_size: int, cos_sin_cache: torch.Tensor, is_neox: bool,
                     value: Optional[torch.Tensor] = None, k_buffer: Optional[torch.Tensor] = None,
                     v_buffer: Optional[torch.Tensor] = None,
                     out_cache_loc: Optional[torch.Tensor] = None) -> None:
    """In place on query/key ([T, H*head_size], row-contiguous views allowed).  With
    value/k_buffer/v_buffer/out_cache_loc also scatters rotated k and v into the KV pool."""
    _gpu(positions, query, key, cos_sin_cache, value, k_buffer, v_buffer, out_cache_loc)
    if query.dim() != 2 or key.dim() != 2 or query.stride(-1) != 1 or key.stride(-1) != 1:
        raise RuntimeError("rotary_embedding needs 2-D row-contiguous q and k (in-place op)")
    if cos_sin_cache.dtype != query.dtype or not cos_sin_cache.is_contiguous():
        raise RuntimeError("cos_sin_cache must be contiguous and in the activation dtype")
    if positions.dtype != torch.int64:
        positions = positions.to(torch.int64)
    positions = positions.contiguous()
    T = query.shape[0]
    Hq, Hkv = query.shape[1] // head_size, key.shape[1] // head_size
    fused = k_buffer is not None
    kv_stride = v_stride = 0
    if fused:
        if value.dim() != 2 or value.stride(-1) != 1:
            raise RuntimeError("fused KV store needs a 2-D row-contiguous value")
        if out_cache_loc.dtype != torch.int64:
            out_cache_loc = out_cache_loc.to(torch.int64)
        _kv_layout(k_buffer, v_buffer, "rotary_embedding (fused KV store)")
        kv_stride, v_stride = k_buffer.stride(0), value.stride(0)
    _check(load().sp_rotary_embedding(
        positions.data_ptr(), query.data_ptr(), key.data_ptr(), cos_sin_cache.data_ptr(), T, Hq, Hkv,
        head_size, cos_sin_cache.shape[1], query.stride(0), key.stride(0), int(is_neox),
        _ptr(value) if fused else None, v_stride, _ptr(k_buffer), _ptr(v_buffer),
        _ptr(out_cache_loc) if fused else None, kv_stride, _dt(query), _stream()),
        "sp_rotary_embedding")


def kv_store(k_buffer: torch.Tensor, v_buffer: torch.Tensor, loc: torch.Tensor,
             cache_k: torch.Tensor, cache_v: torch.Tensor) -> None:
    _gpu(k_buffer, v_buffer, loc, cache_k, cache_v)
    if cache_k.dtype != k_buffer.dtype or cache_v.dtype != v_buffer.dtype:
        raise RuntimeError("kv_store: cache dtype must equal the pool dtype")
    T = cache_k.shape[0]
    k2 = cache_k.reshape(T, -1)
    v2 = cache_v.reshape(T, -1)
    if k2.stride(-1) != 1:
        k2 = k2.contiguous()
    if v2.stride(-1) != 1:
        v2 = v2.contiguous()
    if loc.dtype != torch.int64:
        loc = loc.to(torch.int64)
    loc = loc.contiguous()
    _kv_layout(k_buffer, v_buffer, "kv_store", same_stride=False)
    Hkv, D, Dv = k_buffer.shape[1], k_buffer.shape[2], v_buffer.shape[2]
    _check(load().sp_kv_store(k_buffer.data_ptr(), v_buffer.data_ptr(), loc.data_ptr(), k2.data_ptr(),
                              v2.data_ptr(), T, Hkv, D, Dv, k2.stride(0), v2.stride(0),
                              k_buffer.stride(0), v_buffer.stride(0), _dt(k_buffer), _stream()),
           "sp_kv_store")


def kv_store_fp8(k_buffer: torch.Tensor, v_buffer: torch.Tensor, loc: torch.Tensor, cache_k: torch.Tensor,
                 cache_v: torch.Tensor, k_scale: float = 1.0, v_scale: float = 1.0) -> None:
    """pool[loc] = (cache / scale) rounded to fp8 e5m2; the pool is a uint8 (or float8_e5m2) tensor."""
    _gpu(k_buffer, v_buffer, loc, cache_k, cache_v)
    if k_buffer.dtype not in _FP8_POOL_DTYPES or v_buffer.dtype not in _FP8_POOL_DTYPES:
        raise RuntimeError("kv_store_fp8: the pool must be uint8 / float8_e5m2")
    if cache_k.dtype != cache_v.dtype or cache_k.dtype not in _DTYPES:
        raise RuntimeError("kv_store_fp8: k and v must share a 16/32-bit float dtype")
    T = cache_k.shape[0]
    k2, v2 = cache_k.reshape(T, -1), cache_v.reshape(T, -1)
    if k2.stride(-1) != 1:
        k2 = k2.contiguous()
    if v2.stride(-1) != 1:
        v2 = v2.contiguous()
    loc = loc.to(torch.int64).contiguous()
    _kv_layout(k_buffer, v_buffer, "kv_store_fp8", same_stride=False)
    Hkv, D = k_buffer.shape[1], k_buffer.shape[2]
    if v_buffer.shape[2] != D:
        raise RuntimeError("kv_store_fp8: v_head_dim must equal head_dim")
    _check(load().sp_kv_store_fp8(k_buffer.data_ptr(), v_buffer.data_ptr(), loc.data_ptr(), k2.data_ptr(),
                                  v2.data_ptr(), T, Hkv, D, k2.stride(0), v2.stride(0), k_buffer.stride(0),
                                  v_buffer.stride(0), k_scale, v_scale, _dt(cache_k), _stream()),
           "sp_kv_store_fp8")


# --------------------------------------------------------------------------- index kernels
def write_req_to_token(req_to_token: torch.Tensor, req_pool_indices: torch.Tensor,
                       pre_lens: torch.Tensor, seq_lens: torch.Tensor, extend_lens: torch.Tensor,
                       out_cache_loc: torch.Tensor) -> None:
    _gpu(req_to_token, req_pool_indices, pre_lens, seq_lens, extend_lens, out_cache_loc)
    if req_to_token.dtype != torch.int32:
        raise RuntimeError("req_to_token must be int32")
    args = [t.to(torch.int64).contiguous() for t in
            (req_pool_indices, pre_lens, seq_lens, extend_lens, out_cache_loc)]
    _check(load().sp_write_req_to_token(req_to_token.data_ptr(), req_to_token.stride(0),
                                        *[t.data_ptr() for t in args], req_pool_indices.shape[0],
                                        _stream()), "sp_write_req_to_token")


def compute_position(extend_prefix_lens: torch.Tensor, extend_seq_lens: torch.Tensor,
                     extend_num_tokens: int):
    _gpu(extend_prefix_lens, extend_seq_lens)
    if extend_prefix_lens.dtype != torch.int32 or extend_seq_lens.dtype != torch.int32:
        raise RuntimeError("extend_prefix_lens / extend_seq_lens must be int32")
    bs = extend_seq_lens.shape[0]
    positions = torch.empty(extend_num_tokens, dtype=torch.int64, device=extend_seq_lens.device)
    start = torch.empty(bs, dtype=torch.int32, device=extend_seq_lens.device)
    _check(load().sp_compute_position(positions.data_ptr(), start.data_ptr(),
                                      extend_prefix_lens.contiguous().data_ptr(),
                                      extend_seq_lens.contiguous().data_ptr(), bs, _stream()),
           "sp_compute_position")
    return positions, start


def clamp_position(seq_lens: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _gpu(seq_lens)
    if seq_lens.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("seq_lens must be int32 or int64")
    seq_lens = seq_lens.contiguous()
    if out is None:
        out = torch.empty(seq_lens.shape[0], dtype=torch.int64, device=seq_lens.device)
    _check(load().sp_clamp_position(out.data_ptr(), seq_lens.data_ptr(),
                                    int(seq_lens.dtype == torch.int64), seq_lens.shape[0],
                                    _stream()), "sp_clamp_position")
    return out


# --------------------------------------------------------------------------- attention
def _idx_pair(req_pool_indices: torch.Tensor, seq_lens: torch.Tensor):
    if req_pool_indices.dtype != seq_lens.dtype:
        req_pool_indices = req_pool_indices.to(seq_lens.dtype)
    if seq_lens.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("seq_lens / req_pool_indices must be int32 or int64")
    return req_pool_indices.contiguous(), seq_lens.contiguous(), int(seq_lens.dtype == torch.int64)


def decode_plan_slots(bs: int, max_seq_len: int, chunk: int, kv_tokens: Optional[int] = None) -> int:
    """Partial slots (= work items) a decode step can need: min(bs * ceil(max_seq_len / chunk),
    kv_tokens // chunk + bs), kv_tokens = a bound on sum(seq_lens) (None: the first bound alone)."""
    return int(load().sp_decode_plan_slots(bs, -1 if kv_tokens is None else int(kv_tokens), max_seq_len, chunk))


def decode_workspace_bytes(bs: int, Hq: int, Dv: int, max_seq_len: int, chunk: int,
                           max_slots: Optional[int] = None, ranges: int = 0) -> int:
    """Split workspace for `max_slots` partial slots (default: the static bound bs * ceil(max_seq_len / chunk)) and,
    with `ranges`, for the bs + ranges slots of the range geometry - whichever is larger."""
    if max_slots is None:
        max_slots = decode_plan_slots(bs, max_seq_len, chunk)
    if ranges > 0:
        max_slots = max(max_slots, bs + ranges)
    return int(load().sp_decode_attention_workspace_bytes(max_slots, Hq, Dv))


RANGE_HEADER_WORDS = 4         # [pieces in use, piece length R, ranges, bs] in front of pos[bs + 1] and start[ranges]
RANGE_REQUEST_COST = 16        # positions a request takes on the line beyond its keys (attention_internal.h)


def decode_ranges(Hq: int, Hkv: int, D: int, dtype: torch.dtype, kv_dtype: Optional[torch.dtype] = None) -> int:
    """Pieces the range kernel wants for this shape (sp_decode_ranges): two workgroups per CU (three on a byte pool) over the
    kv heads, a wave per (piece, head); 0 where the range geometry does not apply (fp32, G > 16, D not 64 / 128)."""
    dt = _DTYPES.get(dtype)
    if dt is None:
        return 0
    kv = SP_FP8_E5M2 if kv_dtype in _FP8_POOL_DTYPES else dt
    return int(load().sp_decode_ranges(Hq, Hkv, D, dt, kv))


PLAN_HEADER_WORDS = 4          # [items listed, chunk, items the lengths need, keys the step gathers per kv head]


def _plan_slots(bs: int, max_seq_len: int, chunk: int, max_slots: Optional[int]) -> int:
    return decode_plan_slots(bs, max_seq_len, chunk) if max_slots is None else int(max_slots)


def decode_plan_bytes(bs: int, max_seq_len: int, chunk: int, max_slots: Optional[int] = None, ranges: int = 0) -> int:
    """max_slots = 0 with ranges > 0: a plan without the (request, split) items (range launches only)."""
    return int(load().sp_decode_plan_bytes(bs, _plan_slots(bs, max_seq_len, chunk, max_slots), ranges))


# What each plan buffer was last built with: data_ptr -> (batch size, max_slots, ranges).  The sections of a plan are
# located from these three numbers and a launch has to be given the same ones (include/scratchpad_hip.h, "Plan and launch
# must agree"): the range kernel would do nothing on a mismatch and the item kernels would read another section's words,
# so decode_attention() compares them here, on the host, and raises before anything is launched.  Buffers that were not
# built through decode_plan() (a copy made by hand) are not known and not checked; an entry whose tensor has died is stale
# (the allocator may have handed its address to something else) and is dropped, not trusted.
_BUILT_PLANS: dict = {}            # data_ptr -> (weakref to the plan tensor, (bs, max_slots, ranges))
_BUILT_PLANS_MAX = 4096


def _built_with(plan: torch.Tensor):
    entry = _BUILT_PLANS.get(plan.data_ptr())
    if entry is None:
        return None
    if entry[0]() is None:
        del _BUILT_PLANS[plan.data_ptr()]
        return None
    return entry[1]


def decode_plan(plan: torch.Tensor, seq_lens: torch.Tensor, max_seq_len: int, chunk: int,
                max_slots: Optional[int] = None, ranges: int = 0) -> None:
    """Fill `plan` (int32: [count, chunk, needed, keys | slot0[bs] | (request, split) x max_slots]) for this
    step's lengths.  `max_slots`: the item / partial-slot capacity the launches using this plan are given (default:
    the static bound bs * ceil(max_seq_len / chunk); 0 with ranges > 0: no items, the plan serves range launches only).
    plan[2] > max_slots afterwards means the capacity was too small (see decode_plan_overflow).
    `ranges` > 0 appends the range geometry ([pieces, R, ranges, bs | pos[bs + 1] | start[ranges]],
    include/scratchpad_hip.h) for launches given the same `ranges`."""
    _gpu(plan, seq_lens)
    if plan.dtype != torch.int32 or seq_lens.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("decode_plan: plan must be int32, seq_lens int32/int64")
    seq_lens = seq_lens.contiguous()
    bs = seq_lens.shape[0]
    max_slots = _plan_slots(bs, max_seq_len, chunk, max_slots)
    _check(load().sp_decode_plan(plan.data_ptr(), plan.numel() * 4, seq_lens.data_ptr(),
                                 int(seq_lens.dtype == torch.int64), bs, max_seq_len,
                                 chunk, max_slots, ranges, _stream()), "sp_decode_plan")
    key = plan.data_ptr()
    _BUILT_PLANS.pop(key, None)
    if len(_BUILT_PLANS) >= _BUILT_PLANS_MAX:
        del _BUILT_PLANS[next(iter(_BUILT_PLANS))]
    _BUILT_PLANS[key] = (weakref.ref(plan), (bs, max_slots, int(ranges)))


def decode_plan_overflow(header, max_slots: int) -> Optional[str]:
    """`header`: the first PLAN_HEADER_WORDS ints of a plan, on the host.  None if the plan lists every split the
    lengths need; otherwise the error text (splits were dropped: outputs of this step are wrong)."""
    listed, chunk, needed = int(header[0]), int(header[1]), int(header[2])
    if needed <= max_slots:
        return None
    return (f"decode split plan overflow: the step's seq_lens need {needed} (request, split) items at split size "
            f"{chunk} but the launch was sized for {max_slots} (listed {listed}): the bound on sum(seq_lens) handed to "
            "the attention backend (ForwardBatch.seq_lens_sum) is smaller than the lengths on the device")


def decode_attention(out: torch.Tensor, q: torch.Tensor, k_buffer: torch.Tensor,
                     v_buffer: torch.Tensor, req_to_token: torch.Tensor,
                     req_pool_indices: torch.Tensor, seq_lens: torch.Tensor, sm_scale: float,
                     logit_cap: float, max_seq_len: int, chunk: int, workspace: torch.Tensor,
                     kv_start: Optional[torch.Tensor] = None,
                     plan: Optional[torch.Tensor] = None, k_scale: Optional[float] = None,
                     v_scale: Optional[float] = None, max_slots: Optional[int] = None, ranges: int = 0) -> None:
    """q, out: [bs, Hq, D] (row stride free); buffers [P+1, Hkv, D].  k_scale / v_scale: the
    scales the store divided by (None = 1).  With a plan: `max_slots` = the capacity the plan was built
    for (0: it has no items), `chunk` = the smallest split size the plan may carry (the kernels read the actual one from
    it), `ranges` = the pieces its range section was built for (0: none; the workspace then holds max(max_slots, bs +
    ranges) slots).  Raises if they differ from what decode_plan() built this plan buffer with."""
    _gpu(out, q, k_buffer, v_buffer, req_to_token, req_pool_indices, seq_lens, workspace, kv_start, plan)
    bs, Hq, D = q.shape
    if q.stride(2) != 1 or q.stride(1) != D or out.stride(2) != 1 or out.stride(1) != D:
        raise RuntimeError("decode_attention: q/out must be [bs, Hq, D] with contiguous heads")
    kv_dt = _kv_dt(k_buffer, q, "decode_attention")
    _kv_layout(k_buffer, v_buffer, "decode_attention")
    if v_buffer.dtype != k_buffer.dtype:
        raise RuntimeError("decode_attention: K and V pools must share a dtype")
    req, seq, idx64 = _idx_pair(req_pool_indices, seq_lens)
    if kv_start is not None:
        kv_start = kv_start.to(seq.dtype).contiguous()
    max_slots = _plan_slots(bs, max_seq_len, chunk, max_slots)
    plan_bytes = 0
    if plan is not None:
        plan_bytes = plan.numel() * 4
        built = _built_with(plan)
        if built is not None and built != (bs, max_slots, int(ranges)):
            raise RuntimeError(
                f"decode_attention: the plan was built for (batch size, max_slots, ranges) = {built} and the launch is "
                f"given {(bs, max_slots, int(ranges))}: the plan's sections are located from these numbers, so a launch "
                "must pass the values its plan was built with (sp_decode_plan / sp_decode_attention)")
    _check(load().sp_decode_attention(
        out.data_ptr(), q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(), req_to_token.data_ptr(),
        req_to_token.stride(0), req.data_ptr(), seq.data_ptr(), _ptr(kv_start), idx64, bs, Hq,
        k_buffer.shape[1], D, q.stride(0), out.stride(0), k_buffer.stride(0), sm_scale, logit_cap,
        1.0 if k_scale is None else float(k_scale), 1.0 if v_scale is None else float(v_scale),
        max_seq_len, chunk, max_slots, ranges if plan is not None else 0, workspace.data_ptr(),
        workspace.numel() * workspace.element_size(),
        _ptr(plan), plan_bytes, _dt(q), kv_dt, _stream()), "sp_decode_attention")


def extend_workspace_bytes(num_tokens: int, bs: int, Hq: int, D: int, dtype: torch.dtype) -> int:
    return int(load().sp_extend_attention_workspace_bytes(num_tokens, bs, Hq, D, _DTYPES[dtype]))


def extend_attention(out: torch.Tensor, q: torch.Tensor, k_buffer: torch.Tensor,
                     v_buffer: torch.Tensor, req_to_token: torch.Tensor,
                     req_pool_indices: torch.Tensor, seq_lens: torch.Tensor,
                     extend_seq_lens: torch.Tensor, extend_start_loc: torch.Tensor,
                     sm_scale: float, logit_cap: float, causal: bool, max_extend_len: int,
                     max_seq_len: int, workspace: torch.Tensor,
                     kv_start: Optional[torch.Tensor] = None, window_left: int = -1,
                     k_scale: Optional[float] = None, v_scale: Optional[float] = None,
                     plan: Optional[torch.Tensor] = None) -> None:
    """q, out: [T, Hq, D]; the new tokens' K/V must already be in the pool.  window_left >= 0:
    causal rows see only the window_left keys before their own position (and themselves)."""
    _gpu(out, q, k_buffer, v_buffer, req_to_token, req_pool_indices, seq_lens, extend_seq_lens,
         extend_start_loc, workspace, kv_start, plan)
    if plan is not None and plan.dtype != torch.int32:
        raise RuntimeError("extend_attention: plan must be int32 (extend_plan)")
    T, Hq, D = q.shape
    if q.stride(2) != 1 or q.stride(1) != D or out.stride(2) != 1 or out.stride(1) != D:
        raise RuntimeError("extend_attention: q/out must be [T, Hq, D] with contiguous heads")
    kv_dt = _kv_dt(k_buffer, q, "extend_attention")
    _kv_layout(k_buffer, v_buffer, "extend_attention")
    if v_buffer.dtype != k_buffer.dtype:
        raise RuntimeError("extend_attention: K and V pools must share a dtype")
    if extend_seq_lens.dtype != torch.int32 or extend_start_loc.dtype != torch.int32:
        raise RuntimeError("extend_seq_lens / extend_start_loc must be int32")
    req, seq, idx64 = _idx_pair(req_pool_indices, seq_lens)
    if kv_start is not None:
        kv_start = kv_start.to(seq.dtype).contiguous()
    _check(load().sp_extend_attention(
        out.data_ptr(), q.data_ptr(), k_buffer.data_ptr(), v_buffer.data_ptr(), req_to_token.data_ptr(),
        req_to_token.stride(0), req.data_ptr(), seq.data_ptr(), _ptr(kv_start), idx64,
        extend_seq_lens.contiguous().data_ptr(), extend_start_loc.contiguous().data_ptr(),
        seq.shape[0], T, Hq, k_buffer.shape[1], D, q.stride(0), out.stride(0), k_buffer.stride(0),
        sm_scale, logit_cap, 1.0 if k_scale is None else float(k_scale),
        1.0 if v_scale is None else float(v_scale), int(causal), int(window_left), max_extend_len, max_seq_len, workspace.data_ptr(),
        workspace.numel() * workspace.element_size(), _ptr(plan), 0 if plan is None else plan.numel() * 4,
        _dt(q), kv_dt, _stream()), "sp_extend_attention")


def extend_plan(extend_seq_lens: torch.Tensor, seq_lens: torch.Tensor, num_tokens: int, Hq: int, Hkv: int,
                causal: bool = True, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The (request, row block) work items of an extend step, heaviest first (int32; reuse `out` when it
    is large enough).  Built once per forward, shared by all layers with these head counts."""
    _gpu(extend_seq_lens, seq_lens, out)
    if extend_seq_lens.dtype != torch.int32 or seq_lens.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("extend_plan: extend_seq_lens int32, seq_lens int32/int64")
    bs = extend_seq_lens.shape[0]
    need = int(load().sp_extend_plan_bytes(num_tokens, bs, Hq, Hkv)) // 4
    if out is None or out.numel() < need or out.dtype != torch.int32:
        out = torch.empty(need, dtype=torch.int32, device=extend_seq_lens.device)
    seq = seq_lens.contiguous()
    _check(load().sp_extend_plan(out.data_ptr(), out.numel() * 4, extend_seq_lens.contiguous().data_ptr(),
                                 seq.data_ptr(), int(seq.dtype == torch.int64), bs, num_tokens, Hq, Hkv,
                                 int(causal), _stream()), "sp_extend_plan")
    return out


# --------------------------------------------------------------------------- sampler
def _prob_rows(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dim() != 2 or t.stride(1) != 1:
        raise RuntimeError(f"{what}: expected [batch, vocab] with a contiguous vocab dimension")
    return t


def _opt(t: Optional[torch.Tensor], dtype: torch.dtype, bs: int, what: str):
    if t is None:
        return None
    t = t.reshape(-1)
    if t.shape[0] != bs:
        raise RuntimeError(f"{what}: expected {bs} entries, got {t.shape[0]}")
    return t.to(dtype).contiguous()


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """First maximal index per row -> int64 [bs]."""
    _gpu(logits)
    logits = _prob_rows(logits, "argmax")
    out = torch.empty(logits.shape[0], dtype=torch.int64, device=logits.device)
    _check(load().sp_argmax(logits.data_ptr(), logits.stride(0), logits.shape[0], logits.shape[1],
                            out.data_ptr(), _dt(logits), _stream()), "sp_argmax")
    return out


def argmax_shard(logits: torch.Tensor, cols: int, index_offset: int) -> torch.Tensor:
    """This rank's vocab shard [bs, >= cols] -> int32 [bs, 2] = (fp32 bits of the row maximum over the
    first `cols` columns, global index of its first occurrence)."""
    _gpu(logits)
    logits = _prob_rows(logits, "argmax_shard")
    if not 0 <= cols <= logits.shape[1]:
        raise RuntimeError("argmax_shard: cols out of range")
    out = torch.empty((logits.shape[0], 2), dtype=torch.int32, device=logits.device)
    _check(load().sp_argmax_shard(logits.data_ptr(), logits.stride(0), logits.shape[0], int(cols),
                                  int(index_offset), out.data_ptr(), _dt(logits), _stream()), "sp_argmax_shard")
    return out


def argmax_merge(pairs: torch.Tensor) -> torch.Tensor:
    """pairs: int32 [shards, bs, 2] (rank-major all-gather of argmax_shard outputs) -> int64 [bs]."""
    _gpu(pairs)
    if pairs.dtype != torch.int32 or pairs.dim() != 3 or pairs.shape[2] != 2 or not pairs.is_contiguous():
        raise RuntimeError("argmax_merge: contiguous int32 [shards, bs, 2] expected")
    out = torch.empty(pairs.shape[1], dtype=torch.int64, device=pairs.device)
    _check(load().sp_argmax_merge(pairs.data_ptr(), pairs.shape[0], pairs.shape[1], out.data_ptr(), _stream()),
           "sp_argmax_merge")
    return out


def softmax_temperature_(logits: torch.Tensor, temperatures: Optional[torch.Tensor]) -> torch.Tensor:
    """In place: logits <- softmax(logits / T) (fp32 rows)."""
    _gpu(logits, temperatures)
    logits = _prob_rows(logits, "softmax_temperature_")
    if logits.dtype != torch.float32:
        raise RuntimeError("softmax_temperature_: fp32 logits expected (LogitsProcessor returns fp32)")
    temps = _opt(temperatures, torch.float32, logits.shape[0], "temperatures")
    _check(load().sp_softmax_temperature(logits.data_ptr(), logits.stride(0), _ptr(temps), logits.shape[0],
                                         logits.shape[1], _stream()), "sp_softmax_temperature")
    return logits


def top_k_top_p_min_p_sample(probs: torch.Tensor, top_ks: Optional[torch.Tensor],
                             top_ps: Optional[torch.Tensor], min_ps: Optional[torch.Tensor],
                             uniform: torch.Tensor, return_keep_count: bool = False):
    _gpu(probs, top_ks, top_ps, min_ps, uniform)
    probs = _prob_rows(probs, "top_k_top_p_min_p_sample")
    if probs.dtype != torch.float32:
        raise RuntimeError("top_k_top_p_min_p_sample: fp32 probabilities expected")
    bs, vocab = probs.shape
    ks, ps, ms = (_opt(top_ks, torch.int32, bs, "top_ks"), _opt(top_ps, torch.float32, bs, "top_ps"),
                  _opt(min_ps, torch.float32, bs, "min_ps"))
    u = _opt(uniform, torch.float32, bs, "uniform")
    out = torch.empty(bs, dtype=torch.int64, device=probs.device)
    cnt = torch.empty(bs, dtype=torch.int32, device=probs.device) if return_keep_count else None
    _check(load().sp_top_k_top_p_min_p_sample(probs.data_ptr(), probs.stride(0), _ptr(ks), _ptr(ps), _ptr(ms),
                                              u.data_ptr(), bs, vocab, out.data_ptr(), _ptr(cnt), _stream()),
           "sp_top_k_top_p_min_p_sample")
    return (out, cnt) if return_keep_count else out


def top_k_top_p_min_p_renorm(probs: torch.Tensor, top_ks: Optional[torch.Tensor] = None,
                             top_ps: Optional[torch.Tensor] = None, min_ps: Optional[torch.Tensor] = None,
                             return_keep_count: bool = False):
    _gpu(probs, top_ks, top_ps, min_ps)
    probs = _prob_rows(probs, "top_k_top_p_min_p_renorm")
    if probs.dtype != torch.float32:
        raise RuntimeError("top_k_top_p_min_p_renorm: fp32 probabilities expected")
    bs, vocab = probs.shape
    ks, ps, ms = (_opt(top_ks, torch.int32, bs, "top_ks"), _opt(top_ps, torch.float32, bs, "top_ps"),
                  _opt(min_ps, torch.float32, bs, "min_ps"))
    out = torch.empty_like(probs, memory_format=torch.contiguous_format)
    cnt = torch.empty(bs, dtype=torch.int32, device=probs.device) if return_keep_count else None
    _check(load().sp_top_k_top_p_min_p_renorm(probs.data_ptr(), probs.stride(0), _ptr(ks), _ptr(ps), _ptr(ms),
                                              bs, vocab, out.data_ptr(), out.stride(0), _ptr(cnt), _stream()),
           "sp_top_k_top_p_min_p_renorm")
    return (out, cnt) if return_keep_count else out


# --------------------------------------------------------------------------- small-batch projection
SKINNY_MAX_ROWS = 16
_SKINNY_ON = os.environ.get("SP_SKINNY_GEMM", "1") != "0"


def skinny_gemm_pays(M: int, N: int, K: int) -> bool:
    """Where the weight-streaming kernel measured faster than hipBLASLt on MI355X
    (tools/bench_gemv.py, Llama-3-8B shapes): every lane's x fragment is re-read from L2 per k-step,
    so the win shrinks as rows fill the 16-wide tile and with long rows (down_proj)."""
    if M <= 16 and N * K <= 4096 * 4096:
        return True                       # o_proj-sized: 11 vs 19 us at every M <= 16
    if M <= 2 and K <= 8192:
        return True                       # bs 1-2: qkv 13 vs 19, gate_up 44 vs 60, lm_head 166 vs 179 us
    return M <= 8 and K <= 8192 and N <= 65536


# ---- the row count the library is handed -----------------------------------------------------------------------
# hipBLASLt's kernel choice is erratic in the row count M (tools/bench_gemm_rows.py, device time under graph
# replay, cold weights, MI355X / ROCm 7.2): qkv_proj (N 6144, K 4096) takes 40 us at 256 rows and 28 us at 264;
# down_proj (N 4096, K 14336) 103 us at 192 rows and 59 us at 208.  GEMM rows are independent, so for those
# (shape, M) pairs the product of M rows is computed as the first M rows of an M' > M row product: the input is
# re-viewed over M' rows of its OWN storage (every activation this package allocates carries ROW_SLACK spare rows
# behind it; whatever they hold only reaches output rows that are sliced away), no copy, no extra launch.
#
# The table is a measurement of ONE library build, so it is gated on that build (SP_LIBRARY_ROWS):
#   "table" (default) - the table below, used only while torch / HIP report the versions it was measured on;
#   "auto"            - nothing is assumed: ModelRunner.init_cuda_graphs() times every (projection shape, graph
#                       bucket) against M' = M + 8 .. M + ROW_SLACK on the box it runs on and keeps a substitute
#                       only where it measured faster (calibrate_library_rows); on this build that reproduces the
#                       table, on another library it falls back to M wherever the table's entry does not pay;
#   "0"               - off: every product is run with the row count it was asked for.
ROW_SLACK = 64
_LIBRARY_ROWS_MEASURED_ON = {"torch": "2.10", "hip": "7.0"}      # version prefixes of the build the table is for
_LIBRARY_ROWS_TABLE = {
    (6144, 4096): {136: 176, 144: 176, 152: 176, 192: 200, 224: 232, 256: 264},      # qkv_proj  (8B)
    (4096, 4096): {96: 104, 192: 208},                                                # o_proj
    (28672, 4096): {16: 40, 48: 56, 80: 96},                                          # gate_up_proj
    (4096, 14336): {72: 80, 96: 112, 128: 136, 160: 208, 192: 208},                   # down_proj
    # Llama-3-70B shards at TP = 8 (profiles/r02_gemm_rows_70b_tp8.txt); nothing to gain at config 4's 128 rows
    (7168, 8192): {192: 200, 224: 232, 256: 264},                                     # gate_up_proj / 8
    (8192, 3584): {192: 208, 224: 232, 256: 264},                                     # down_proj / 8
    (1280, 8192): {64: 72},                                                           # qkv_proj / 8
}
SLACK_MAX_ROWS = 256          # decode-sized steps only; larger products are exactly F.linear


def library_versions_match() -> bool:
    hip = getattr(torch.version, "hip", None) or ""
    return (torch.__version__.startswith(_LIBRARY_ROWS_MEASURED_ON["torch"])
            and hip.startswith(_LIBRARY_ROWS_MEASURED_ON["hip"]))


def _library_rows_mode() -> str:
    m = os.environ.get("SP_LIBRARY_ROWS", "table").lower()
    return {"1": "table", "on": "table", "off": "0"}.get(m, m)


_LIBROWS_MODE = _library_rows_mode()
if _LIBROWS_MODE == "table" and library_versions_match():
    _LIBRARY_ROWS = {k: dict(v) for k, v in _LIBRARY_ROWS_TABLE.items()}
else:
    _LIBRARY_ROWS = {}        # off, another library build, or "auto" before calibrate_library_rows() has run
_LIBROWS_USED = {}            # (N, K, M) -> M' of every substitution made so far (reported by bench.py)


def library_rows(M: int, N: int, K: int) -> int:
    """rows to hand the library GEMM for an M-row product of shape (N, K): M, or the measured better M' > M"""
    return _LIBRARY_ROWS.get((N, K), {}).get(M, M)


def library_rows_report() -> dict:
    """What bench.py records: the mode, whether the version gate passed, and every substitution that was used."""
    return {"mode": _LIBROWS_MODE, "versions_match": library_versions_match(),
            "measured_on": dict(_LIBRARY_ROWS_MEASURED_ON),
            "running_on": {"torch": torch.__version__, "hip": getattr(torch.version, "hip", None)},
            "substituted": {f"N={n} K={k} M={m}": mp for (n, k, m), mp in sorted(_LIBROWS_USED.items())}}


def _time_mm(x: torch.Tensor, weights, reps: int = 3) -> float:
    """device microseconds of x @ W.T, one call per weight captured into a HIP graph (the weights of different
    layers are cycled so that no call finds its weights in L2 / the Infinity Cache, as in the decode step)"""
    outs = [torch.empty((x.shape[0], w.shape[0]), dtype=x.dtype, device=x.device) for w in weights[:2]]
    st = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        for i, w in enumerate(weights):
            torch.mm(x, w.t(), out=outs[i % 2])
        st.synchronize()
        with torch.cuda.graph(g, stream=st, capture_error_mode="thread_local"):
            for i, w in enumerate(weights):
                torch.mm(x, w.t(), out=outs[i % 2])
    torch.cuda.synchronize()
    g.replay()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (reps * len(weights)) * 1e3


def calibrate_library_rows(weights_by_shape, rows, min_gain: float = 0.05, step: int = 8) -> dict:
    """SP_LIBRARY_ROWS=auto.  weights_by_shape: {(N, K): [weight tensors of that shape]} (the model's own
    projections); rows: the batch-size buckets of the decode graphs.  Every (shape, M) is timed against
    M' = M + step .. M + ROW_SLACK; a substitute is kept only where it is at least `min_gain` faster than M
    itself ON THIS BOX.  Replaces the active table and returns it."""
    global _LIBRARY_ROWS
    found = {}
    for (N, K), ws in weights_by_shape.items():
        ws = list(ws)[:8]
        if not ws or ws[0].dtype not in (torch.float16, torch.bfloat16) or not ws[0].is_cuda:
            continue
        xbuf = torch.randn((max(rows) + ROW_SLACK, K), device=ws[0].device).to(ws[0].dtype) * 0.1
        cache = {}

        def t_of(m):
            if m not in cache:
                cache[m] = _time_mm(xbuf[:m], ws)
            return cache[m]

        for M in sorted(set(rows)):
            if not 16 < M <= SLACK_MAX_ROWS:        # <= 16 rows: the skinny kernel's territory
                continue
            base = t_of(M)
            best_t, best_m = base, M
            for Mp in range((M // step + 1) * step, M + ROW_SLACK + 1, step):
                t = t_of(Mp)
                if t < best_t:
                    best_t, best_m = t, Mp
            if best_m != M and best_t <= base * (1.0 - min_gain):
                found.setdefault((N, K), {})[M] = best_m
    _LIBRARY_ROWS = found
    return found


def empty_rows(rows: int, cols: int, dtype, device, zero: bool = False) -> torch.Tensor:
    """[rows, cols] activation with ROW_SLACK readable spare rows behind it in the same allocation"""
    full = (torch.zeros if zero else torch.empty)((rows + ROW_SLACK, cols), dtype=dtype, device=device)
    return full[:rows]


def extend_rows(x: torch.Tensor, rows: int) -> Optional[torch.Tensor]:
    """x re-viewed over `rows` >= x.shape[0] rows of its own storage, or None if the storage ends before"""
    if rows <= x.shape[0]:
        return x
    if x.dim() != 2 or x.stride(1) != 1 or x.stride(0) < x.shape[1]:
        return None
    last = x.storage_offset() + (rows - 1) * x.stride(0) + x.shape[1]
    if last * x.element_size() > x.untyped_storage().nbytes():
        return None
    return torch.as_strided(x, (rows, x.shape[1]), (x.stride(0), 1), x.storage_offset())


_SILU_LINEAR_ON = os.environ.get("SP_SKINNY_SILU", "1") != "0"
# rows up to which the fused form is used.  Measured (round 4, bench.py --ctx 1024, HIP-graph replay, ms/step fused vs
# projection + activation launch): bs 1 3.977 vs 4.006, bs 8 4.469 vs 4.579, bs 16 5.052 vs 4.698 - at 16 rows the
# merged projection is faster on the library (61 vs 68 us) and the activation launch it saves costs ~1 us under replay
SILU_FUSED_MAX_ROWS = 8


def linear_silu_mul(x: torch.Tensor, gate_up_weight: torch.Tensor, any_rows: bool = False) -> Optional[torch.Tensor]:
    """SiluAndMul(x @ gate_up_weight.T) as ONE launch (sp_gemm_skinny, epilogue 1) for a step of at most
    SILU_FUSED_MAX_ROWS tokens (any_rows: up to the kernel's 16): x [M, K], gate_up_weight [2 I, K] (gate rows first),
    result [M, I].  Bit for bit the skinny projection followed by silu_and_mul.  None when the shape is not taken (the
    caller runs the two steps)."""
    if not (_SKINNY_ON and _SILU_LINEAR_ON and x.is_cuda and x.dim() == 2 and gate_up_weight.dim() == 2
            and 0 < x.shape[0] <= (SKINNY_MAX_ROWS if any_rows else SILU_FUSED_MAX_ROWS)
            and gate_up_weight.shape[1] == x.shape[1]
            and gate_up_weight.shape[0] % 16 == 0
            and x.dtype in (torch.float16, torch.bfloat16) and gate_up_weight.dtype == x.dtype
            and x.shape[1] % 32 == 0 and x.stride(1) == 1 and gate_up_weight.stride(1) == 1
            and x.stride(0) % 8 == 0 and gate_up_weight.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and gate_up_weight.data_ptr() % 16 == 0):
        return None
    M, K = x.shape
    inter = gate_up_weight.shape[0] // 2
    out = empty_rows(M, inter, x.dtype, x.device)
    _check(load().sp_gemm_skinny(out.data_ptr(), x.data_ptr(), gate_up_weight.data_ptr(), M, inter, K, x.stride(0),
                                 gate_up_weight.stride(0), out.stride(0), 1, _dt(x), _stream()), "sp_gemm_skinny(silu)")
    return out


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """x @ weight.T.  Small-batch 16-bit products go to the weight-streaming kernel
    (sp_gemm_skinny) where it pays; everything else is the library GEMM - exactly F.linear, except
    that a product of at most SLACK_MAX_ROWS rows whose (shape, rows) is in the active library_rows
    table is computed over more rows than asked for (first M rows returned; rows are independent)."""
    if (_SKINNY_ON and x.is_cuda and x.dim() == 2 and 0 < x.shape[0] <= SKINNY_MAX_ROWS
            and skinny_gemm_pays(x.shape[0], weight.shape[0], x.shape[1])
            and x.dtype in (torch.float16, torch.bfloat16) and weight.dtype == x.dtype
            and x.shape[1] % 32 == 0 and x.stride(1) == 1 and weight.stride(1) == 1
            and x.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0):
        M, K = x.shape
        N = weight.shape[0]
        out = empty_rows(M, N, x.dtype, x.device)
        _check(load().sp_gemm_skinny(out.data_ptr(), x.data_ptr(), weight.data_ptr(), M, N, K, x.stride(0),
                                     weight.stride(0), out.stride(0), 0, _dt(x), _stream()), "sp_gemm_skinny")
        return out
    if (_LIBRARY_ROWS and x.is_cuda and x.dim() == 2 and 0 < x.shape[0] <= SLACK_MAX_ROWS and weight.dim() == 2
            and x.dtype in (torch.float16, torch.bfloat16) and weight.dtype == x.dtype and x.stride(1) == 1):
        M, K = x.shape
        N = weight.shape[0]
        Mp = library_rows(M, N, K)
        xe = extend_rows(x, Mp) if Mp > M else x
        if xe is None:                      # producer without spare rows (e.g. the embedding): run as asked
            xe, Mp = x, M
        # the output carries spare rows only where another measured projection may consume it (one whose input
        # width is this output's width); anything else - the LM head above all - is exactly F.linear
        if Mp > M or _feeds_a_measured_shape(N):
            if Mp > M:
                _LIBROWS_USED[(N, K, M)] = Mp
            out = torch.empty((Mp + ROW_SLACK, N), dtype=x.dtype, device=x.device)
            torch.mm(xe, weight.t(), out=out[:Mp])
            return out[:M]
    return torch.nn.functional.linear(x, weight)


def _feeds_a_measured_shape(width: int) -> bool:
    return any(k == width for (_n, k) in _LIBRARY_ROWS)


# --------------------------------------------------------------------------- per-sequence state, latent attention, experts
class SeqParams:
    """The header's SP_SEQ_PARAMS of one step, built once per forward (``from_forward_batch``) and handed to every kernel
    that reads or writes per-request state.  Holds the tensors, so the pointers stay valid while it lives."""

    def __init__(self, req_pool_indices: torch.Tensor, seq_lens: torch.Tensor, extend_seq_lens=None,
                 extend_prefix_lens=None, extend_start_loc=None, token_req=None):
        _gpu(req_pool_indices, seq_lens, extend_seq_lens, extend_prefix_lens, extend_start_loc, token_req)
        if req_pool_indices.dtype not in (torch.int32, torch.int64):
            raise RuntimeError("req_pool_indices must be int32 or int64")
        if seq_lens.dtype != req_pool_indices.dtype:
            seq_lens = seq_lens.to(req_pool_indices.dtype)
        self.req_pool_indices, self.seq_lens = req_pool_indices.contiguous(), seq_lens.contiguous()
        ext = (extend_seq_lens, extend_prefix_lens, extend_start_loc, token_req)
        if any(t is not None for t in ext):
            if any(t is None or t.dtype != torch.int32 for t in ext):
                raise RuntimeError("a multi-token step needs extend_seq_lens, extend_prefix_lens, extend_start_loc and "
                                   "token_req, all int32")
            ext = tuple(t.contiguous() for t in ext)
        self.extend_seq_lens, self.extend_prefix_lens, self.extend_start_loc, self.token_req = ext
        self.batch_size = int(self.req_pool_indices.shape[0])
        self.num_tokens = self.batch_size if token_req is None else int(self.token_req.shape[0])
        self.args = [self.req_pool_indices.data_ptr(), self.seq_lens.data_ptr(), _ptr(self.extend_seq_lens),
                     _ptr(self.extend_prefix_lens), _ptr(self.extend_start_loc), _ptr(self.token_req),
                     int(self.req_pool_indices.dtype == torch.int64), self.batch_size]

    @classmethod
    def from_forward_batch(cls, fb) -> "SeqParams":
        if fb.forward_mode.is_decode():
            return cls(fb.req_pool_indices, fb.seq_lens)
        bs = fb.batch_size
        token_req = torch.repeat_interleave(torch.arange(bs, dtype=torch.int32, device=fb.extend_seq_lens.device),
                                            fb.extend_seq_lens.long(), output_size=fb.extend_num_tokens)
        return cls(fb.req_pool_indices, fb.seq_lens, fb.extend_seq_lens, fb.extend_prefix_lens, fb.extend_start_loc,
                   token_req)


def _f32(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
        raise RuntimeError(f"{what} must be a contiguous fp32 device tensor")
    return t


def _mat(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dim() != 2 or t.stride(1) != 1:
        raise RuntimeError(f"{what} must be [rows, n] with a contiguous last dimension, got {tuple(t.shape)} {tuple(t.stride())}")
    return t


def bigram_rows(ids: torch.Tensor, last_token: torch.Tensor, seq: SeqParams, buckets: int, mul_prev: int,
                mul_cur: int) -> torch.Tensor:
    _gpu(ids, last_token)
    if ids.dtype != torch.int64 or last_token.dtype != torch.int64 or ids.shape[0] != seq.num_tokens:
        raise RuntimeError("bigram_rows: ids [num_tokens] and last_token must be int64")
    rows = torch.empty(ids.shape[0], dtype=torch.int32, device=ids.device)
    _check(load().sp_bigram_rows(rows.data_ptr(), ids.data_ptr(), last_token.data_ptr(), ids.shape[0], *seq.args,
                                 buckets, mul_prev, mul_cur, _stream()), "sp_bigram_rows")
    return rows


def save_last_token(last_token: torch.Tensor, ids: torch.Tensor, seq: SeqParams) -> None:
    _check(load().sp_save_last_token(last_token.data_ptr(), ids.data_ptr(), *seq.args, _stream()), "sp_save_last_token")


def save_last_rows(state: torch.Tensor, x: torch.Tensor, seq: SeqParams) -> None:
    _f32(state, "state")
    _mat(x, "x")
    if x.dtype != torch.float32 or state.shape[-1] != x.shape[1] or x.shape[0] != seq.num_tokens:
        raise RuntimeError("save_last_rows: x [num_tokens, width] fp32, state [slots, width]")
    _check(load().sp_save_last_rows(state.data_ptr(), state.stride(0), x.data_ptr(), x.stride(0), x.shape[1], *seq.args,
                                    _stream()), "sp_save_last_rows")


def embed_bigram_norm(embed: torch.Tensor, bigram: torch.Tensor, ids: torch.Tensor, rows: torch.Tensor,
                      gain: torch.Tensor, eps: float):
    """(x fp32 [T, W], the same in the tables' dtype)"""
    _gpu(embed, bigram, ids, rows)
    _f32(gain, "gain")
    if embed.dtype != bigram.dtype or embed.shape[1] != bigram.shape[1] or not embed.is_contiguous() or not bigram.is_contiguous():
        raise RuntimeError("embed_bigram_norm: tables must share dtype and width and be contiguous")
    T, W = ids.shape[0], embed.shape[1]
    x = torch.empty((T, W), dtype=torch.float32, device=embed.device)
    lo = x if embed.dtype == torch.float32 else empty_rows(T, W, embed.dtype, embed.device)
    _check(load().sp_embed_bigram_norm(x.data_ptr(), None if lo is x else lo.data_ptr(), embed.data_ptr(), bigram.data_ptr(),
                                       ids.data_ptr(), rows.data_ptr(), gain.data_ptr(), T, W, x.stride(0), lo.stride(0),
                                       eps, _dt(embed), _stream()), "sp_embed_bigram_norm")
    return x, lo


def add_scalar_norm(x: torch.Tensor, y: torch.Tensor, gain: torch.Tensor, eps: float, want_lo: bool = True):
    """x += y / rms(y) * gain in place (x fp32); returns x in y's dtype for the next projection (x itself when fp32)"""
    _mat(x, "x"), _mat(y, "y"), _f32(gain, "gain")
    if x.dtype != torch.float32 or x.shape != y.shape:
        raise RuntimeError("add_scalar_norm: x fp32 [T, W], y [T, W]")
    lo = None
    if want_lo and y.dtype != torch.float32:
        lo = empty_rows(x.shape[0], x.shape[1], y.dtype, x.device)
    _check(load().sp_add_scalar_norm(x.data_ptr(), _ptr(lo), y.data_ptr(), gain.data_ptr(), x.shape[0], x.shape[1],
                                     x.stride(0), 0 if lo is None else lo.stride(0), y.stride(0), eps, _dt(y), _stream()),
           "sp_add_scalar_norm")
    return x if lo is None else lo


def scalar_norm(x: torch.Tensor, gain: torch.Tensor, eps: float, dtype: torch.dtype) -> torch.Tensor:
    _mat(x, "x"), _f32(gain, "gain")
    if x.dtype != torch.float32:
        raise RuntimeError("scalar_norm: x must be fp32")
    out = empty_rows(x.shape[0], x.shape[1], dtype, x.device)
    _check(load().sp_scalar_norm(out.data_ptr(), x.data_ptr(), gain.data_ptr(), x.shape[0], x.shape[1], x.stride(0),
                                 out.stride(0), eps, _DTYPES[dtype], _stream()), "sp_scalar_norm")
    return out


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    _mat(z, "z"), _f32(coef, "coef")
    out = empty_rows(z.shape[0], z.shape[1], z.dtype, z.device)
    _check(load().sp_polynorm(out.data_ptr(), z.data_ptr(), coef.data_ptr(), z.shape[0], z.shape[1], z.stride(0),
                              out.stride(0), eps, _dt(z), _stream()), "sp_polynorm")
    return out


def gate_heads(o: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """o [H, T, D] contiguous, g [T, H] -> [T, H * D] = o * sigmoid(g) per head"""
    _mat(g, "g")
    if o.dim() != 3 or not o.is_contiguous() or g.shape != (o.shape[1], o.shape[0]) or g.dtype != o.dtype:
        raise RuntimeError("gate_heads: o [H, T, D] contiguous, g [T, H] of the same dtype")
    H, T, D = o.shape
    out = empty_rows(T, H * D, o.dtype, o.device)
    _check(load().sp_gate_heads(out.data_ptr(), o.data_ptr(), g.data_ptr(), T, H, D, g.stride(0), _dt(o), _stream()),
           "sp_gate_heads")
    return out


def token_shift(x: torch.Tensor, mu: torch.Tensor, shift_state: torch.Tensor, seq: SeqParams, dtype: torch.dtype) -> torch.Tensor:
    """[mixes, T, W] in dtype: x[t] + (x[t-1] - x[t]) * mu[m]"""
    _mat(x, "x"), _f32(mu, "mu"), _f32(shift_state, "shift_state")
    if x.dtype != torch.float32 or mu.shape[1] != x.shape[1] or shift_state.shape[1] != x.shape[1] or x.shape[0] != seq.num_tokens:
        raise RuntimeError("token_shift: x fp32 [num_tokens, W], mu [mixes, W], shift_state [slots, W]")
    out = torch.empty((mu.shape[0] * x.shape[0] + ROW_SLACK, x.shape[1]), dtype=dtype, device=x.device)
    _check(load().sp_token_shift(out.data_ptr(), x.data_ptr(), mu.data_ptr(), shift_state.data_ptr(), shift_state.stride(0),
                                 x.shape[0], x.shape[1], mu.shape[0], x.stride(0), *seq.args, _DTYPES[dtype], _stream()),
           "sp_token_shift")
    return out[:mu.shape[0] * x.shape[0]].view(mu.shape[0], x.shape[0], x.shape[1])


def wkv_decay(a: torch.Tensor, w2t: torch.Tensor, w0: torch.Tensor) -> torch.Tensor:
    _mat(a, "a"), _f32(w2t, "w2t"), _f32(w0, "w0")
    if w2t.shape[0] != a.shape[1] or w0.shape[0] != w2t.shape[1]:
        raise RuntimeError("wkv_decay: a [T, rank], w2t [rank, channels], w0 [channels]")
    out = torch.empty((a.shape[0], w2t.shape[1]), dtype=torch.float32, device=a.device)
    _check(load().sp_wkv_decay(out.data_ptr(), a.data_ptr(), w2t.data_ptr(), w0.data_ptr(), a.shape[0], w2t.shape[1],
                               w2t.shape[0], a.stride(0), _dt(a), _stream()), "sp_wkv_decay")
    return out


def wkv_recurrence(r, k, v, g, decay, u, norm_w, state, seq: SeqParams, heads: int, dim: int, eps: float) -> torch.Tensor:
    for name, t in (("r", r), ("k", k), ("v", v), ("g", g)):
        _mat(t, name)
        if t.dtype != r.dtype or t.shape != (seq.num_tokens, heads * dim):
            raise RuntimeError(f"wkv_recurrence: {name} must be [num_tokens, heads * dim] of one dtype")
    _f32(decay, "decay"), _f32(u, "u"), _f32(norm_w, "norm_w"), _f32(state, "state")
    if decay.shape != r.shape or u.numel() != heads * dim or norm_w.numel() != heads * dim or \
            state.shape[1:] != (heads, dim, dim):
        raise RuntimeError("wkv_recurrence: decay [T, H*D], u [H, D], norm_w [H*D], state [slots, H, D, D]")
    out = empty_rows(r.shape[0], heads * dim, r.dtype, r.device)
    _check(load().sp_wkv_recurrence(out.data_ptr(), r.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), decay.data_ptr(),
                                    u.data_ptr(), norm_w.data_ptr(), state.data_ptr(), state.stride(0), heads, dim,
                                    r.stride(0), k.stride(0), v.stride(0), g.stride(0), out.stride(0), eps, *seq.args,
                                    _dt(r), _stream()), "sp_wkv_recurrence")
    return out


def rotary_interleaved(x: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor, mag: float, offset: int = 0) -> None:
    """in place on x [T, H, n]: the pairs of x[..., offset : offset + 2 * len(freq)]"""
    _f32(freq, "freq")
    if x.dim() != 3 or x.stride(2) != 1 or positions.dtype != torch.int64 or offset + 2 * freq.shape[0] > x.shape[2]:
        raise RuntimeError("rotary_interleaved: x [T, H, n] with contiguous last dimension, int64 positions")
    _check(load().sp_rotary_interleaved(x.data_ptr(), positions.data_ptr(), freq.data_ptr(), mag, x.shape[0], x.shape[1],
                                        2 * freq.shape[0], x.stride(0), x.stride(1), offset, _dt(x), _stream()),
           "sp_rotary_interleaved")


def latent_kv_store(pool: torch.Tensor, dkv: torch.Tensor, norm_w: torch.Tensor, positions: torch.Tensor,
                    freq: torch.Tensor, mag: float, loc: torch.Tensor, rank: int, eps: float) -> None:
    _mat(pool, "pool"), _mat(dkv, "dkv"), _f32(norm_w, "norm_w"), _f32(freq, "freq")
    rot_dim = dkv.shape[1] - rank
    if pool.dtype != dkv.dtype or pool.shape[1] != dkv.shape[1] or norm_w.shape[0] != rank or rot_dim < 2 * freq.shape[0] \
            or loc.dtype != torch.int64 or positions.dtype != torch.int64 or loc.shape[0] != dkv.shape[0]:
        raise RuntimeError("latent_kv_store: pool [P, rank + rot], dkv [T, rank + rot] of one dtype, int64 loc / positions")
    _check(load().sp_latent_kv_store(pool.data_ptr(), pool.stride(0), dkv.data_ptr(), dkv.stride(0), norm_w.data_ptr(),
                                     positions.data_ptr(), freq.data_ptr(), mag, loc.data_ptr(), dkv.shape[0], rank, rot_dim,
                                     2 * freq.shape[0], eps, _dt(dkv), _stream()), "sp_latent_kv_store")


def latent_attention(q_lat: torch.Tensor, q_rot: torch.Tensor, pool: torch.Tensor, req_to_token: torch.Tensor,
                     seq: SeqParams, scale: float) -> torch.Tensor:
    """q_lat [H, T, rank] contiguous; q_rot [T, H, rot] (a view: strides are taken); pool [P, rank + rot]; -> [H, T, rank]"""
    _mat(pool, "pool")
    H, T, rank = q_lat.shape
    if not q_lat.is_contiguous() or q_rot.dim() != 3 or q_rot.stride(2) != 1 or q_rot.shape[:2] != (T, H) or \
            pool.shape[1] != rank + q_rot.shape[2] or q_lat.dtype != pool.dtype or q_rot.dtype != pool.dtype or \
            req_to_token.dtype != torch.int32 or T != seq.num_tokens:
        raise RuntimeError("latent_attention: shapes / dtypes do not fit")
    out = torch.empty((H, T, rank), dtype=q_lat.dtype, device=q_lat.device)
    _check(load().sp_latent_attention(out.data_ptr(), q_lat.data_ptr(), q_rot.data_ptr(), pool.data_ptr(), pool.stride(0),
                                      req_to_token.data_ptr(), req_to_token.stride(0), T, H, rank, q_rot.shape[2],
                                      q_rot.stride(0), q_rot.stride(1), scale, *seq.args, _dt(q_lat), _stream()),
           "sp_latent_attention")
    return out


def moe_route(x: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int):
    """(ids int32 [T, top], weights fp32 [T, top])"""
    _mat(x, "x"), _f32(router, "router"), _f32(correction, "correction")
    T, E = x.shape[0], router.shape[0]
    ids = torch.empty((T, top), dtype=torch.int32, device=x.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=x.device)
    _check(load().sp_moe_route(ids.data_ptr(), weights.data_ptr(), x.data_ptr(), x.stride(0), router.data_ptr(),
                               correction.data_ptr(), T, x.shape[1], E, top, groups, keep, _dt(x), _stream()), "sp_moe_route")
    return ids, weights


def moe_align(ids: torch.Tensor, experts: int):
    """(offsets [E + 1], order [P], place [P]) int32: the (token, expert) pairs ordered by expert"""
    P = ids.numel()
    offsets = torch.empty(experts + 1, dtype=torch.int32, device=ids.device)
    order = torch.empty(P, dtype=torch.int32, device=ids.device)
    place = torch.empty(P, dtype=torch.int32, device=ids.device)
    _check(load().sp_moe_align(offsets.data_ptr(), order.data_ptr(), place.data_ptr(), ids.data_ptr(), P, experts, _stream()),
           "sp_moe_align")
    return offsets, order, place


def moe_grouped_gemm(a: torch.Tensor, w: torch.Tensor, offsets: torch.Tensor, pairs: int, order: Optional[torch.Tensor] = None,
                     row_div: int = 1) -> torch.Tensor:
    """out [pairs, N]: row pos = w[expert of pos] @ a[order[pos] // row_div] (a[pos] without order); w [E, N, K]"""
    _mat(a, "a")
    if w.dim() != 3 or not w.is_contiguous() or w.dtype != a.dtype or w.shape[2] != a.shape[1]:
        raise RuntimeError("moe_grouped_gemm: w [E, N, K] contiguous of a's dtype")
    E, N, K = w.shape
    out = torch.empty((pairs, N), dtype=a.dtype, device=a.device)
    _check(load().sp_moe_grouped_gemm(out.data_ptr(), a.data_ptr(), w.data_ptr(), offsets.data_ptr(), _ptr(order), row_div,
                                      pairs, N, K, E, a.stride(0), out.stride(0), _dt(a), _stream()), "sp_moe_grouped_gemm")
    return out


def moe_glu(gu: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    if gu.dim() != 2 or not gu.is_contiguous() or gu.shape[1] % 2:
        raise RuntimeError("moe_glu: gu [P, 2 * ff] contiguous")
    out = torch.empty((gu.shape[0], gu.shape[1] // 2), dtype=gu.dtype, device=gu.device)
    _check(load().sp_moe_glu(out.data_ptr(), gu.data_ptr(), gu.shape[0], gu.shape[1] // 2, limit, alpha, _dt(gu), _stream()),
           "sp_moe_glu")
    return out


def moe_combine(z: torch.Tensor, place: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
    T, top = weights.shape
    if z.dim() != 2 or not z.is_contiguous() or z.shape[0] != T * top:
        raise RuntimeError("moe_combine: z [T * top, W] contiguous")
    out = empty_rows(T, z.shape[1], z.dtype, z.device)
    _check(load().sp_moe_combine(out.data_ptr(), z.data_ptr(), place.data_ptr(), weights.data_ptr(), T, z.shape[1], top,
                                 out.stride(0), _dt(z), _stream()), "sp_moe_combine")
    return out


# --------------------------------------------------------------------------- fp32 stream with token shift, windowed attention, scans
def moe_route_softmax(x: torch.Tensor, router: torch.Tensor, top: int, scale: float, bias: Optional[torch.Tensor] = None,
                      renorm: bool = False):
    """(ids int32 [T, top], weights fp32 [T, top]): fp32 logits router x (+ bias), the largest softmax scores, times scale;
    ``renorm``: divided by their sum (the softmax over the chosen logits only)"""
    logits = small_linear_f32(x, router, bias)
    T, E = logits.shape
    ids = torch.empty((T, top), dtype=torch.int32, device=x.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=x.device)
    _check(load().sp_moe_softmax_topk(ids.data_ptr(), weights.data_ptr(), logits.data_ptr(), T, E, top, scale, int(renorm),
                                      _stream()), "sp_moe_softmax_topk")
    return ids, weights


def embed_scale(embed: torch.Tensor, ids: torch.Tensor, scale: float) -> torch.Tensor:
    """fp32 [T, W] = embed[ids] * scale"""
    _gpu(embed, ids)
    if ids.dtype != torch.int64 or embed.dim() != 2 or not embed.is_contiguous():
        raise RuntimeError("embed_scale: int64 ids, contiguous table [vocab, width]")
    x = torch.empty((ids.shape[0], embed.shape[1]), dtype=torch.float32, device=embed.device)
    _check(load().sp_embed_scale(x.data_ptr(), x.stride(0), embed.data_ptr(), ids.data_ptr(), ids.shape[0], embed.shape[1],
                                 embed.shape[0], scale, _dt(embed), _stream()), "sp_embed_scale")
    return x


def norm_shift(x: torch.Tensor, weight: torch.Tensor, eps: float, dtype: torch.dtype, mu: Optional[torch.Tensor] = None,
               state: Optional[torch.Tensor] = None, seq: Optional[SeqParams] = None, want_h: bool = True):
    """(h, hs) in dtype: h = x / rms(x) * weight, hs = h + (h[t-1] - h) * mu (None without mu).  With mu, the request's
    saved h (``state`` [slots, W] fp32) precedes a step's first row and is replaced by the step's last h."""
    _mat(x, "x"), _f32(weight, "weight")
    if x.dtype != torch.float32 or weight.shape[0] != x.shape[1]:
        raise RuntimeError("norm_shift: x fp32 [T, W], weight [W]")
    T, W = x.shape
    h = empty_rows(T, W, dtype, x.device) if want_h or mu is None else None
    hs = None
    if mu is not None:
        _f32(mu, "mu"), _f32(state, "state")
        if seq is None or seq.num_tokens != T or state.shape[1] != W or mu.shape[0] != W:
            raise RuntimeError("norm_shift: mu [W], state [slots, W] and the step's SeqParams go together")
        hs = empty_rows(T, W, dtype, x.device)
    stride = (h if h is not None else hs).stride(0)
    args = seq.args if seq is not None else [None] * 6 + [0, 0]
    _check(load().sp_norm_shift(_ptr(h), _ptr(hs), stride, x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(mu), _ptr(state),
                                0 if state is None else state.stride(0), T, W, eps, *args, _DTYPES[dtype], _stream()),
           "sp_norm_shift")
    if mu is not None:
        _check(load().sp_norm_save_last(state.data_ptr(), state.stride(0), x.data_ptr(), x.stride(0), weight.data_ptr(), W, eps,
                                        *seq.args, _stream()), "sp_norm_save_last")
    return h, hs


def stream_add(x: torch.Tensor, a: torch.Tensor, b: Optional[torch.Tensor] = None, c: Optional[torch.Tensor] = None) -> None:
    """x += a + b + c in place (x fp32)"""
    _mat(x, "x")
    if x.dtype != torch.float32:
        raise RuntimeError("stream_add: x must be fp32")
    for t in (a, b, c):
        if t is not None and (_mat(t, "addend").shape != x.shape or t.dtype != a.dtype):
            raise RuntimeError("stream_add: addends [T, W] of one dtype")
    _check(load().sp_stream_add(x.data_ptr(), x.stride(0), a.data_ptr(), a.stride(0), _ptr(b), 0 if b is None else b.stride(0),
                                _ptr(c), 0 if c is None else c.stride(0), x.shape[0], x.shape[1], _dt(a), _stream()),
           "sp_stream_add")


def qkv_rotary_store(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor,
                     positions: torch.Tensor, loc: torch.Tensor, freq: Optional[torch.Tensor], mag: float, heads: int,
                     kv_heads: int, dim: int, vdim: int, eps: float, adjacent: bool = False, norm_values: bool = True,
                     q_bias: Optional[torch.Tensor] = None, k_bias: Optional[torch.Tensor] = None,
                     v_bias: Optional[torch.Tensor] = None, qk_norm: bool = False, q_head_scale: Optional[torch.Tensor] = None,
                     q_temp: Optional[Tuple[float, int]] = None, v_first: Optional[torch.Tensor] = None,
                     v_mix: Optional[torch.Tensor] = None) -> None:
    """q [T, heads * dim] rotated in place; k rotated, v (head-normed unless ``norm_values`` is off) into the pools' rows
    loc (views: strides are taken).  ``adjacent``: coordinate 2i pairs with 2i + 1 instead of i with i + dims / 2.  fp32
    biases, where given, are added before the rotation / the norm.  ``qk_norm``: q and k divided per head by their root
    mean square after the rotation; ``q_head_scale`` fp32 [heads] and ``q_temp`` = (coef, every): q times the head's number
    and times 1 + coef ln(floor((position + 1) / every) + 1); ``v_first`` (another layer's value pool) with ``v_mix`` (fp32,
    one number): the stored value is (1 - v_mix) v + v_mix v_first[loc]."""
    for name, t, n in (("q", q, heads * dim), ("k", k, kv_heads * dim), ("v", v, kv_heads * vdim)):
        if _mat(t, name).shape[1] != n or t.dtype != q.dtype or t.shape[0] != q.shape[0]:
            raise RuntimeError(f"qkv_rotary_store: {name} must be [T, {n}]")
    if kpool.dtype != q.dtype or vpool.dtype != q.dtype or _mat(kpool, "kpool").shape[1] != kv_heads * dim or \
            _mat(vpool, "vpool").shape[1] != kv_heads * vdim:
        raise RuntimeError("qkv_rotary_store: pools [P, kv_heads * dim] / [P, kv_heads * vdim] of q's dtype")
    if positions.dtype != torch.int64 or loc.dtype != torch.int64 or loc.shape[0] != q.shape[0] or positions.shape[0] != q.shape[0]:
        raise RuntimeError("qkv_rotary_store: int64 positions and loc, one per row")
    for name, t, n in (("q_bias", q_bias, heads * dim), ("k_bias", k_bias, kv_heads * dim), ("v_bias", v_bias, kv_heads * vdim)):
        if t is not None and _f32(t, name).numel() != n:
            raise RuntimeError(f"qkv_rotary_store: {name} must hold {n} values")
    dims = 0 if freq is None else 2 * _f32(freq, "freq").shape[0]
    if q_head_scale is not None and _f32(q_head_scale, "q_head_scale").numel() != heads:
        raise RuntimeError("qkv_rotary_store: q_head_scale must hold one value per query head")
    if v_first is not None and (v_mix is None or _f32(v_mix, "v_mix").numel() != 1 or v_first.shape != vpool.shape or
                                v_first.dtype != vpool.dtype):
        raise RuntimeError("qkv_rotary_store: v_first must mirror vpool and come with v_mix (one fp32 number)")
    coef, every = q_temp if q_temp else (0.0, 0)
    _check(load().sp_qkv_rotary_store(q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
                                      kpool.data_ptr(), kpool.stride(0), vpool.data_ptr(), vpool.stride(0), positions.data_ptr(),
                                      loc.data_ptr(), _ptr(freq), mag, _ptr(q_bias), _ptr(k_bias), _ptr(v_bias), q.shape[0],
                                      heads, kv_heads, dim, vdim, dims, int(adjacent), int(norm_values), eps, int(qk_norm),
                                      _ptr(q_head_scale), float(coef), int(every), _ptr(v_first),
                                      0 if v_first is None else v_first.stride(0), _ptr(v_mix), _dt(q), _stream()),
           "sp_qkv_rotary_store")


def pool_blocks(kpooled: torch.Tensor, vpooled: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor,
                req_to_token: torch.Tensor, seq: SeqParams, block: int) -> None:
    if kpooled.shape != kpool.shape or vpooled.shape != vpool.shape or kpooled.dtype != kpool.dtype or \
            kpooled.stride(0) != kpool.stride(0) or vpooled.stride(0) != vpool.stride(0) or req_to_token.dtype != torch.int32:
        raise RuntimeError("pool_blocks: pooled buffers must mirror the token buffers")
    _check(load().sp_pool_blocks(kpooled.data_ptr(), vpooled.data_ptr(), kpool.data_ptr(), vpool.data_ptr(), kpool.stride(0),
                                 vpool.stride(0), req_to_token.data_ptr(), req_to_token.stride(0), seq.num_tokens,
                                 kpool.shape[1], vpool.shape[1], block, *seq.args, _dt(kpool), _stream()), "sp_pool_blocks")


def window_attention(q: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, kpooled: Optional[torch.Tensor],
                     vpooled: Optional[torch.Tensor], req_to_token: torch.Tensor, seq: SeqParams, heads: int, kv_heads: int,
                     dim: int, vdim: int, window: int, block: int, scale: float, matrix: bool = True,
                     sinks: Optional[torch.Tensor] = None, softcap: float = 0.0, sigmoid_weights: bool = False,
                     head_bias: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [T, heads * dim] (rotated) -> [T, heads * vdim]; matrix=False keeps 16-bit prompt portions off the matrix-core
    kernel (comparisons); sinks fp32 [heads]: one more term exp(sink) in every softmax's denominator; softcap > 0: scores
    capped as softcap tanh(score / softcap); sigmoid_weights: a visible key's weight is sigmoid(score + head_bias[head]),
    not normalised; gate [T, heads * vdim] (a view): the result times sigmoid(gate)"""
    _mat(q, "q"), _mat(kpool, "kpool"), _mat(vpool, "vpool")
    T = q.shape[0]
    if q.shape[1] != heads * dim or kpool.shape[1] != kv_heads * dim or vpool.shape[1] != kv_heads * vdim or \
            kpool.dtype != q.dtype or vpool.dtype != q.dtype or req_to_token.dtype != torch.int32 or T != seq.num_tokens:
        raise RuntimeError("window_attention: shapes / dtypes do not fit")
    if kpooled is not None and (kpooled.stride(0) != kpool.stride(0) or vpooled.stride(0) != vpool.stride(0)):
        raise RuntimeError("window_attention: pooled buffers must mirror the token buffers")
    if sinks is not None and _f32(sinks, "sinks").numel() != heads:
        raise RuntimeError("window_attention: sinks must hold one value per query head")
    if head_bias is not None and _f32(head_bias, "head_bias").numel() != heads:
        raise RuntimeError("window_attention: head_bias must hold one value per query head")
    if gate is not None and (_mat(gate, "gate").shape != (T, heads * vdim) or gate.dtype != q.dtype):
        raise RuntimeError("window_attention: gate must be [T, heads * vdim] of q's dtype")
    out = empty_rows(T, heads * vdim, q.dtype, q.device)
    _check(load().sp_window_attention(out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), kpool.data_ptr(),
                                      vpool.data_ptr(), _ptr(kpooled), _ptr(vpooled), kpool.stride(0), vpool.stride(0),
                                      req_to_token.data_ptr(), req_to_token.stride(0), T, heads, kv_heads, dim, vdim,
                                      window, block, scale, _ptr(sinks), float(softcap or 0.0), int(sigmoid_weights),
                                      _ptr(head_bias), _ptr(gate), 0 if gate is None else gate.stride(0), int(matrix),
                                      *seq.args, _dt(q), _stream()),
           "sp_window_attention")
    return out


SMALL_LINEAR_OWN_ROWS = 64      # up to this many rows small_linear_f32 runs on the library's own kernel


def small_linear_f32(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 [T, n] = x @ weight.T + bias with fp32 weights, accumulation and output (gates and step sizes of recurrences)"""
    _mat(x, "x"), _f32(weight, "weight")
    if weight.dim() != 2 or weight.shape[1] != x.shape[1] or (bias is not None and _f32(bias, "bias").shape[0] != weight.shape[0]):
        raise RuntimeError("small_linear_f32: weight [n, k], bias [n]")
    if x.shape[0] > SMALL_LINEAR_OWN_ROWS:
        # many rows: the own kernel reads the weight rows again for every token; the library's fp32 product tiles them
        return torch.nn.functional.linear(x.to(torch.float32), weight, bias)
    out = torch.empty((x.shape[0], weight.shape[0]), dtype=torch.float32, device=x.device)
    _check(load().sp_small_linear_f32(out.data_ptr(), x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), x.shape[0],
                                      x.shape[1], weight.shape[0], _dt(x), _stream()), "sp_small_linear_f32")
    return out


def causal_conv_silu(u: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
                     seq: SeqParams) -> torch.Tensor:
    """u [T, C] (a view: its row stride is taken) -> silu(conv) [T, C]; state [slots, taps - 1, C] fp32 is read and moved on"""
    _mat(u, "u"), _f32(weight, "weight"), _f32(state, "state")
    C, taps = weight.shape
    if u.shape[1] != C or u.shape[0] != seq.num_tokens or state.shape[1:] != (max(taps - 1, 0), C) or \
            (bias is not None and _f32(bias, "bias").shape[0] != C):
        raise RuntimeError("causal_conv_silu: u [num_tokens, C], weight [C, taps], state [slots, taps - 1, C]")
    out = empty_rows(u.shape[0], C, u.dtype, u.device)
    _check(load().sp_causal_conv_silu(out.data_ptr(), out.stride(0), u.data_ptr(), u.stride(0), weight.data_ptr(), _ptr(bias),
                                      state.data_ptr(), state.stride(0), u.shape[0], C, taps, *seq.args, _dt(u), _stream()),
           "sp_causal_conv_silu")
    return out


def mamba2_scan(xbc: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, A_log: torch.Tensor, D: torch.Tensor,
                state: torch.Tensor, seq: SeqParams, heads: int, groups: int, state_size: int, vdim: int) -> torch.Tensor:
    """xbc [T, heads * vdim + 2 * groups * state_size] -> y fp32 [T, heads * vdim]; state [slots, heads, state_size, vdim]"""
    _mat(xbc, "xbc"), _f32(dt_raw, "dt_raw"), _f32(dt_bias, "dt_bias"), _f32(A_log, "A_log"), _f32(D, "D"), _f32(state, "state")
    inner = heads * vdim
    if xbc.shape != (seq.num_tokens, inner + 2 * groups * state_size) or dt_raw.shape != (seq.num_tokens, heads) or \
            state.shape[1:] != (heads, state_size, vdim) or dt_bias.numel() != heads or A_log.numel() != heads or D.numel() != heads:
        raise RuntimeError("mamba2_scan: shapes do not fit")
    y = torch.empty((xbc.shape[0], inner), dtype=torch.float32, device=xbc.device)
    _check(load().sp_mamba2_scan(y.data_ptr(), y.stride(0), xbc.data_ptr(), xbc.stride(0), dt_raw.data_ptr(), dt_bias.data_ptr(),
                                 A_log.data_ptr(), D.data_ptr(), state.data_ptr(), state.stride(0), heads, groups, state_size,
                                 vdim, *seq.args, _dt(xbc), _stream()), "sp_mamba2_scan")
    return y


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, parts: int, eps: float) -> torch.Tensor:
    """(y * silu(z)) normed in `parts` equal parts, times weight; y fp32, z (a view) and the result in z's dtype"""
    _mat(y, "y"), _mat(z, "z"), _f32(weight, "weight")
    if y.dtype != torch.float32 or y.shape != z.shape or weight.shape[0] != y.shape[1] or y.shape[1] % parts:
        raise RuntimeError("gated_group_norm: y fp32 [T, n], z [T, n], weight [n], n divisible by parts")
    out = empty_rows(y.shape[0], y.shape[1], z.dtype, y.device)
    _check(load().sp_gated_group_norm(out.data_ptr(), out.stride(0), y.data_ptr(), y.stride(0), z.data_ptr(), z.stride(0),
                                      weight.data_ptr(), y.shape[0], y.shape[1], parts, eps, _dt(z), _stream()),
           "sp_gated_group_norm")
    return out


def mlstm_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, ipre: torch.Tensor, fpre: torch.Tensor,
               norm_w: torch.Tensor, S: torch.Tensor, n: torch.Tensor, m: torch.Tensor, seq: SeqParams, heads: int, dim: int,
               vdim: int, cap: float, eps: float) -> torch.Tensor:
    """q, k [T, heads * dim], v, g [T, heads * vdim] (views) -> [T, heads * vdim]; states S [slots, heads, dim, vdim],
    n [slots, heads, dim], m [slots, heads] fp32"""
    T = seq.num_tokens
    for name, t, w in (("q", q, heads * dim), ("k", k, heads * dim), ("v", v, heads * vdim), ("g", g, heads * vdim)):
        if _mat(t, name).shape != (T, w) or t.dtype != q.dtype:
            raise RuntimeError(f"mlstm_scan: {name} must be [num_tokens, {w}] of one dtype")
    _f32(ipre, "ipre"), _f32(fpre, "fpre"), _f32(norm_w, "norm_w"), _f32(S, "S"), _f32(n, "n"), _f32(m, "m")
    if ipre.shape != (T, heads) or fpre.shape != (T, heads) or norm_w.numel() != heads * vdim or \
            S.shape[1:] != (heads, dim, vdim) or n.shape[1:] != (heads, dim) or m.shape[1:] != (heads,):
        raise RuntimeError("mlstm_scan: gate or state shapes do not fit")
    out = empty_rows(T, heads * vdim, q.dtype, q.device)
    _check(load().sp_mlstm_scan(out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0),
                                v.data_ptr(), v.stride(0), g.data_ptr(), g.stride(0), ipre.data_ptr(), fpre.data_ptr(),
                                norm_w.data_ptr(), S.data_ptr(), S.stride(0), n.data_ptr(), n.stride(0), m.data_ptr(),
                                m.stride(0), heads, dim, vdim, cap, eps, *seq.args, _dt(q), _stream()), "sp_mlstm_scan")
    return out


# --------------------------------------------------------------------------- gated normed sublayer results, delta rule, forget-write scan
def gated_add_norm(x: torch.Tensor, a: torch.Tensor, weight: torch.Tensor, eps: float, gate: Optional[torch.Tensor] = None,
                   gate_bias: Optional[torch.Tensor] = None, b: Optional[torch.Tensor] = None, wa: Optional[torch.Tensor] = None,
                   wb: Optional[torch.Tensor] = None, extra: Optional[torch.Tensor] = None,
                   next_weight: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """x fp32 [T, W] += N(y * sigmoid(gate + gate_bias)) * weight in place, y = a, or (N(a) wa + N(b) wb) / 2 with a second
    branch; then x += extra (fp32); with ``next_weight`` returns N(x) * next_weight in a's dtype (the next sublayer's
    input).  a, b, gate may be views (their row strides are taken)."""
    _mat(x, "x"), _mat(a, "a"), _f32(weight, "weight")
    T, W = x.shape
    if x.dtype != torch.float32 or a.shape != (T, W) or weight.numel() != W:
        raise RuntimeError("gated_add_norm: x fp32 [T, W], a [T, W], weight [W]")
    for name, t in (("b", b), ("gate", gate)):
        if t is not None and (_mat(t, name).shape != (T, W) or t.dtype != a.dtype):
            raise RuntimeError(f"gated_add_norm: {name} must be [T, W] of a's dtype")
    if b is not None and (wa is None or wb is None or _f32(wa, "wa").numel() != W or _f32(wb, "wb").numel() != W):
        raise RuntimeError("gated_add_norm: two branches need their norm weights wa, wb [W]")
    if gate_bias is not None and _f32(gate_bias, "gate_bias").numel() != W:
        raise RuntimeError("gated_add_norm: gate_bias [W]")
    if extra is not None and (_mat(extra, "extra").shape != (T, W) or extra.dtype != torch.float32):
        raise RuntimeError("gated_add_norm: extra fp32 [T, W]")
    nxt = None
    if next_weight is not None:
        if _f32(next_weight, "next_weight").numel() != W:
            raise RuntimeError("gated_add_norm: next_weight [W]")
        nxt = empty_rows(T, W, a.dtype, x.device)
    _check(load().sp_gated_add_norm(x.data_ptr(), x.stride(0), a.data_ptr(), a.stride(0), _ptr(wa), _ptr(b),
                                    0 if b is None else b.stride(0), _ptr(wb), _ptr(gate), 0 if gate is None else gate.stride(0),
                                    _ptr(gate_bias), weight.data_ptr(), _ptr(extra), 0 if extra is None else extra.stride(0),
                                    _ptr(nxt), 0 if nxt is None else nxt.stride(0), _ptr(next_weight), T, W, eps, _dt(a),
                                    _stream()), "sp_gated_add_norm")
    return nxt


def relu_square(x: torch.Tensor) -> torch.Tensor:
    """max(x, 0)^2 of x [T, d] (a view: its row stride is taken)"""
    _mat(x, "x")
    out = empty_rows(x.shape[0], x.shape[1], x.dtype, x.device)
    _check(load().sp_relu_square(out.data_ptr(), x.data_ptr(), x.shape[0], x.shape[1], x.stride(0), out.stride(0), _dt(x),
                                 _stream()), "sp_relu_square")
    return out


def scale_softcap(logits: torch.Tensor, scale: float, cap: float) -> torch.Tensor:
    """fp32 [rows, n] = cap * tanh(logits * scale / cap) (cap 0 or less: logits * scale)"""
    _mat(logits, "logits")
    out = torch.empty(logits.shape, dtype=torch.float32, device=logits.device)
    _check(load().sp_scale_softcap(out.data_ptr(), out.stride(0), logits.data_ptr(), logits.stride(0), logits.shape[0],
                                   logits.shape[1], scale, cap or 0.0, _dt(logits), _stream()), "sp_scale_softcap")
    return out


def delta_gates(p: torch.Tensor, w2t: torch.Tensor, w0: torch.Tensor, apre: torch.Tensor, a_bias: torch.Tensor, rate: float):
    """(decay, remove) fp32 [T, channels]: exp(-rate * sigmoid(tanh(p) w2t + w0)) and sigmoid(apre + a_bias)"""
    _mat(p, "p"), _mat(apre, "apre"), _f32(w2t, "w2t"), _f32(w0, "w0"), _f32(a_bias, "a_bias")
    T, n = apre.shape
    if w2t.shape != (p.shape[1], n) or w0.numel() != n or a_bias.numel() != n or p.shape[0] != T or p.dtype != apre.dtype:
        raise RuntimeError("delta_gates: p [T, rank], w2t [rank, channels], w0, a_bias [channels], apre [T, channels]")
    decay = torch.empty((T, n), dtype=torch.float32, device=p.device)
    remove = torch.empty((T, n), dtype=torch.float32, device=p.device)
    _check(load().sp_delta_gates(decay.data_ptr(), remove.data_ptr(), p.data_ptr(), p.stride(0), w2t.data_ptr(), w0.data_ptr(),
                                 apre.data_ptr(), apre.stride(0), a_bias.data_ptr(), T, n, p.shape[1], rate, _dt(p), _stream()),
           "sp_delta_gates")
    return decay, remove


def delta_recurrence(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, decay: torch.Tensor,
                     remove: torch.Tensor, norm_w: torch.Tensor, state: torch.Tensor, seq: SeqParams, heads: int, dim: int,
                     eps: float) -> torch.Tensor:
    """r, k, v, g [T, heads * dim] (views) -> [T, heads * dim]; state [slots, heads, dim, dim] fp32 is read and moved on"""
    T, n = seq.num_tokens, heads * dim
    for name, t in (("r", r), ("k", k), ("v", v), ("g", g)):
        if _mat(t, name).shape != (T, n) or t.dtype != r.dtype:
            raise RuntimeError(f"delta_recurrence: {name} must be [num_tokens, heads * dim] of one dtype")
    _f32(decay, "decay"), _f32(remove, "remove"), _f32(norm_w, "norm_w"), _f32(state, "state")
    if decay.shape != (T, n) or remove.shape != (T, n) or norm_w.numel() != n or state.shape[1:] != (heads, dim, dim):
        raise RuntimeError("delta_recurrence: decay, remove [T, H*D], norm_w [H*D], state [slots, H, D, D]")
    out = empty_rows(T, n, r.dtype, r.device)
    _check(load().sp_delta_recurrence(out.data_ptr(), out.stride(0), r.data_ptr(), r.stride(0), k.data_ptr(), k.stride(0),
                                      v.data_ptr(), v.stride(0), g.data_ptr(), g.stride(0), decay.data_ptr(), remove.data_ptr(),
                                      norm_w.data_ptr(), state.data_ptr(), state.stride(0), heads, dim, eps, *seq.args,
                                      _dt(r), _stream()), "sp_delta_recurrence")
    return out


def hgrn2_scan(qpre: torch.Tensor, fpre: torch.Tensor, v: torch.Tensor, f_bias: torch.Tensor, lower: torch.Tensor,
               norm_w: torch.Tensor, state: torch.Tensor, seq: SeqParams, heads: int, dim: int, vdim: int, eps: float) -> torch.Tensor:
    """qpre, fpre [T, heads * dim], v [T, heads * vdim] (views) -> [T, heads * vdim]; state [slots, heads, dim, vdim] fp32"""
    T = seq.num_tokens
    for name, t, w in (("qpre", qpre, heads * dim), ("fpre", fpre, heads * dim), ("v", v, heads * vdim)):
        if _mat(t, name).shape != (T, w) or t.dtype != qpre.dtype:
            raise RuntimeError(f"hgrn2_scan: {name} must be [num_tokens, {w}] of one dtype")
    _f32(f_bias, "f_bias"), _f32(lower, "lower"), _f32(norm_w, "norm_w"), _f32(state, "state")
    if f_bias.numel() != heads * dim or lower.numel() != heads * dim or norm_w.numel() != vdim or \
            state.shape[1:] != (heads, dim, vdim):
        raise RuntimeError("hgrn2_scan: f_bias, lower [H*D], norm_w [vdim], state [slots, H, D, vdim]")
    out = empty_rows(T, heads * vdim, qpre.dtype, qpre.device)
    _check(load().sp_hgrn2_scan(out.data_ptr(), out.stride(0), qpre.data_ptr(), qpre.stride(0), fpre.data_ptr(), fpre.stride(0),
                                v.data_ptr(), v.stride(0), f_bias.data_ptr(), lower.data_ptr(), norm_w.data_ptr(),
                                state.data_ptr(), state.stride(0), heads, dim, vdim, eps, *seq.args, _dt(qpre), _stream()),
           "sp_hgrn2_scan")
    return out


# --------------------------------------------------------------------------- norm in groups, channel-gated delta rule
def add_group_norm(x: torch.Tensor, a: Optional[torch.Tensor], groups: int, eps: float, dtype: torch.dtype,
                   b: Optional[torch.Tensor] = None, wa: Optional[torch.Tensor] = None, wb: Optional[torch.Tensor] = None,
                   next_weight: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """x fp32 [T, W] += a (or (N(a) wa + N(b) wb) / 2 with a second branch; nothing when a is None) in place; with
    ``next_weight`` returns GN(x) * next_weight in ``dtype``: every one of ``groups`` equal parts of the row divided by its
    own root mean square.  a, b may be views (their row strides are taken)."""
    _mat(x, "x")
    T, W = x.shape
    if x.dtype != torch.float32 or W % groups:
        raise RuntimeError("add_group_norm: x fp32 [T, W], W divisible by groups")
    for name, t in (("a", a), ("b", b)):
        if t is not None and (_mat(t, name).shape != (T, W) or t.dtype != dtype):
            raise RuntimeError(f"add_group_norm: {name} must be [T, W] of the given dtype")
    if b is not None and (a is None or wa is None or wb is None or _f32(wa, "wa").numel() != W or _f32(wb, "wb").numel() != W):
        raise RuntimeError("add_group_norm: two branches need their norm weights wa, wb [W]")
    nxt = None
    if next_weight is not None:
        if _f32(next_weight, "next_weight").numel() != W:
            raise RuntimeError("add_group_norm: next_weight [W]")
        nxt = empty_rows(T, W, dtype, x.device)
    elif a is None:
        return None
    _check(load().sp_add_group_norm(x.data_ptr(), x.stride(0), _ptr(a), 0 if a is None else a.stride(0), _ptr(wa), _ptr(b),
                                    0 if b is None else b.stride(0), _ptr(wb), _ptr(nxt), 0 if nxt is None else nxt.stride(0),
                                    _ptr(next_weight), T, W, groups, eps, _DTYPES[dtype], _stream()), "sp_add_group_norm")
    return nxt


def lowrank_gate(p: torch.Tensor, w2t: torch.Tensor, bias: Optional[torch.Tensor], act: str,
                 A_log: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 [T, channels]: z = p w2t + bias (p [T, rank] a view, w2t fp32 [rank, channels]); act "decay":
    exp(-exp(A_log[head]) softplus(z)) with channels / len(A_log) channels per head, act "sigmoid": sigmoid(z)"""
    _mat(p, "p"), _f32(w2t, "w2t")
    T, (rank, n) = p.shape[0], w2t.shape
    if p.shape[1] != rank or (bias is not None and _f32(bias, "bias").numel() != n) or act not in ("decay", "sigmoid"):
        raise RuntimeError("lowrank_gate: p [T, rank], w2t [rank, channels], bias [channels]")
    per = 1
    if act == "decay":
        if A_log is None or n % _f32(A_log, "A_log").numel():
            raise RuntimeError("lowrank_gate: the decay needs A_log [heads], heads dividing the channels")
        per = n // A_log.numel()
    out = torch.empty((T, n), dtype=torch.float32, device=p.device)
    _check(load().sp_lowrank_gate(out.data_ptr(), p.data_ptr(), p.stride(0), w2t.data_ptr(), _ptr(bias), _ptr(A_log), T, n, rank,
                                  per, 0 if act == "decay" else 1, _dt(p), _stream()), "sp_lowrank_gate")
    return out


def gated_delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, bpre: torch.Tensor, decay: torch.Tensor,
                     gate: torch.Tensor, norm_w: torch.Tensor, state: torch.Tensor, seq: SeqParams, heads: int, kv_heads: int,
                     dim: int, vdim: int, eps: float) -> torch.Tensor:
    """q, k [T, kv_heads * dim], v [T, heads * vdim], bpre [T, heads] (views) -> [T, heads * vdim]; decay fp32
    [T, heads * dim], gate fp32 [T, heads * vdim]; state [slots, heads, dim, vdim] fp32 is read and moved on"""
    T = seq.num_tokens
    for name, t, w in (("q", q, kv_heads * dim), ("k", k, kv_heads * dim), ("v", v, heads * vdim), ("bpre", bpre, heads)):
        if _mat(t, name).shape != (T, w) or t.dtype != q.dtype:
            raise RuntimeError(f"gated_delta_scan: {name} must be [num_tokens, {w}] of one dtype")
    _f32(decay, "decay"), _f32(gate, "gate"), _f32(norm_w, "norm_w"), _f32(state, "state")
    if decay.shape != (T, heads * dim) or gate.shape != (T, heads * vdim) or norm_w.numel() != vdim or \
            state.shape[1:] != (heads, dim, vdim) or not decay.is_contiguous() or not gate.is_contiguous():
        raise RuntimeError("gated_delta_scan: decay [T, H*D], gate [T, H*Dv], norm_w [Dv], state [slots, H, D, Dv]")
    out = empty_rows(T, heads * vdim, q.dtype, q.device)
    _check(load().sp_gated_delta_scan(out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0),
                                      v.data_ptr(), v.stride(0), bpre.data_ptr(), bpre.stride(0), decay.data_ptr(),
                                      gate.data_ptr(), norm_w.data_ptr(), state.data_ptr(), state.stride(0), heads, kv_heads,
                                      dim, vdim, eps, *seq.args, _dt(q), _stream()), "sp_gated_delta_scan")
    return out
