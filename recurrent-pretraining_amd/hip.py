"""ctypes binding of libraven_hip.so (the C ABI declared in include/raven_hip.h).

PyTorch is used only for device memory and streams: tensors cross the boundary as raw device
pointers plus sizes, and every launch goes to torch's current HIP stream.  There is no fallback:
if the library is missing or a call fails, an exception is raised.
"""

from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import torch

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libraven_hip.so")

F32, BF16 = 0, 1
_DTYPES = {torch.float32: F32, torch.bfloat16: BF16}


class RavenHipError(RuntimeError):
    pass


class Dims(C.Structure):
    _fields_ = [("n_embd", C.c_int32), ("n_heads", C.c_int32), ("head_dim", C.c_int32),
                ("intermediate", C.c_int32), ("eps", C.c_float), ("dtype", C.c_int32)]


class BlockWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in
                ("norm_1", "norm_2", "norm_3", "norm_4", "wqkv", "qk_bias", "proj", "fc", "mlp_proj")]


class KVCache(C.Structure):
    _fields_ = [("k", C.c_void_p), ("v", C.c_void_p), ("n_slots", C.c_int32), ("batch", C.c_int32),
                ("t_max", C.c_int32), ("lookup_mode", C.c_int32), ("steps_present", C.c_void_p),
                ("core_slot0", C.c_int32)]


class PagedKV(C.Structure):
    _fields_ = [("k_caches", C.POINTER(C.c_void_p)), ("v_caches", C.POINTER(C.c_void_p)), ("block_table", C.c_void_p),
                ("seq_lens", C.c_void_p), ("max_blocks", C.c_int32), ("block_size", C.c_int32), ("max_seq_len", C.c_int32),
                ("kv_layout", C.c_int32)]


PAGED_NHD, PAGED_HND = 0, 1


def _paged_dims(cache: torch.Tensor, layout: int):
    """(block_size, n_heads, head_dim) of a paged cache tensor: [blocks, block_size, nh, hd] (NHD) or [blocks, nh, block_size, hd]."""
    if layout == PAGED_NHD:
        _, bs, nh, hd = cache.shape
    elif layout == PAGED_HND:
        _, nh, bs, hd = cache.shape
    else:
        raise RavenHipError(f"unknown paged layout {layout}")
    return bs, nh, hd


LOOKUP_NONE, LOOKUP_SKIP, LOOKUP_LATEST, LOOKUP_ALWAYS_LAST = 0, 1, 2, 3


# name -> (restype, argtypes); kept in one table so the export test can walk it
_VP, _I32, _I64, _F, _SZ = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_size_t
SIGNATURES = {
    "raven_version": (C.c_int, []),
    "raven_arch": (C.c_char_p, []),
    "raven_last_error": (C.c_char_p, []),
    "raven_set_tuning": (C.c_int, [C.c_char_p, _I32]),
    "raven_rmsnorm_residual": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _I64, _I32, _F, _I32, _VP]),
    "raven_gemm": (C.c_int, [_VP, _VP, _VP, _VP, _I32, _I32, _I32, _I32, _I32, _VP]),
    "raven_adapter_gemm_concat": (C.c_int, [_VP, _VP, _VP, _VP, _I32, _I32, _I32, _I32, _I32, _VP]),
    "raven_gemm_swiglu": (C.c_int, [_VP, _VP, _VP, _I32, _I32, _I32, _I32, _VP]),
    "raven_packed_weight_bytes": (_I64, [_I32, _I32]),
    "raven_register_packed_weight": (C.c_int, [_VP, _I32, _I32, _VP, _VP]),
    "raven_unregister_packed_weight": (C.c_int, [_VP]),
    "raven_linear_workspace_bytes": (_SZ, [_I32, _I32]),
    "raven_linear": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _VP, _SZ, _VP]),
    "raven_exit_logit_stats": (C.c_int, [_VP, _VP, _VP, _I32, _I32, _I32, _VP]),
    "raven_exit_latent_stats": (C.c_int, [_VP, _VP, _VP, _VP, _I32, _I32, _I32, _VP]),
    "raven_paged_kv_append": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _I32, _I32, _I32, _I32, _I32, _I32, _VP]),
    "raven_paged_decode_attention": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _VP, _SZ,
                                               _VP]),
    "raven_paged_qkv_attention_decode": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _I32,
                                                   _VP, _SZ, _VP]),
    "raven_gemv_fused": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _I32, _I32, _I32, _F, _I32, _I32, _I32, _VP]),
    "raven_qkv_bias_rope_cache_append": (C.c_int, [_VP, _VP, _VP, _VP, C.POINTER(KVCache), _I32, _I32, _I32, _I32,
                                                   _VP, _I32, _I32, _I32, _VP]),
    "raven_decode_attention_workspace_bytes": (_SZ, [_I32, _I32, _I32]),
    "raven_decode_attention": (C.c_int, [_VP, _VP, C.POINTER(KVCache), _I32, _I32, _I32, _I32, _VP, _I32, _I32, _I32,
                                         _VP, _SZ, _VP]),
    "raven_qkv_attention_decode": (C.c_int, [_VP, _VP, _VP, _VP, C.POINTER(KVCache), _I32, _I32, _I32, _VP, _I32, _I32,
                                             _I32, _VP, _SZ, _VP]),
    "raven_qkv_attention_decode_static_scratch_bytes": (_SZ, []),
    "raven_qkv_attention_decode_static": (C.c_int, [_VP, _VP, _VP, _VP, C.POINTER(KVCache), _I32, _I32, _I32, _VP, _I32, _I32, _I32, _VP]),
    "raven_prefill_attention": (C.c_int, [_VP, _VP, C.POINTER(KVCache), _I32, _I32, _I32, _I32, _VP, _I32, _I32, _I32, _VP]),
    "raven_swiglu": (C.c_int, [_VP, _VP, _I32, _I32, _I32, _VP]),
    "raven_noise_mix": (C.c_int, [_VP, _VP, _VP, _I64, _F, _F, _F, _I32, _VP]),
    "raven_embed": (C.c_int, [_VP, _VP, _VP, _I32, _I32, _I64, _F, _I32, _VP]),
    "raven_argmax": (C.c_int, [_VP, _VP, _I32, _I64, _VP]),
    "raven_advance_pos": (C.c_int, [_VP, _I32, _VP]),
    "raven_block_workspace_bytes": (_SZ, [C.POINTER(Dims), _I32]),
    "raven_sandwich_block": (C.c_int, [C.POINTER(Dims), C.POINTER(BlockWeights), _VP, _VP, _VP, _VP,
                                       C.POINTER(KVCache), _I32, _I32, _I32, _I32, _VP, _VP, _SZ, _VP]),
    "raven_core_iteration": (C.c_int, [C.POINTER(Dims), _VP, C.POINTER(BlockWeights), _I32, _VP, _VP, _VP, _VP, _VP,
                                       C.POINTER(KVCache), _I32, _I32, _I32, _I32, _VP, _VP, _SZ, _VP]),
    "raven_core_iterations": (C.c_int, [C.POINTER(Dims), _VP, C.POINTER(BlockWeights), _I32, _VP, _VP, _VP, _VP, _VP,
                                        C.POINTER(KVCache), C.POINTER(C.c_int32), _I32, _I32, _I32, _I32, _VP, _VP, _SZ, _VP]),
    "raven_paged_qkv_rope_append": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _I32, _I32, _I32, _I32, _I32, _I32, _VP]),
    "raven_paged_prefill_attention": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _VP]),
    "raven_paged_decode_blocks": (C.c_int, [C.POINTER(Dims), _VP, C.POINTER(BlockWeights), _I32, _VP, _VP, _VP, _VP, _VP,
                                            C.POINTER(PagedKV), _I32, _I32, _VP, _SZ, _VP]),
}

_lib: Optional[C.CDLL] = None


def load() -> C.CDLL:
    """Loads the library (once).  Raises when it has not been built: there is no other code path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RavenHipError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as e; e.build()'` "
                "(hipcc, gfx950).  This package has no CPU or PyTorch fallback.")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().raven_last_error().decode("utf-8", "replace")
        raise RavenHipError(f"{what} failed (code {rc}): {msg}")


def set_tuning(key: str, value: int) -> None:
    _check(load().raven_set_tuning(key.encode(), int(value)), "raven_set_tuning")


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPES[dt]
    except KeyError:
        raise RavenHipError(f"unsupported dtype {dt}: the kernels take float32 and bfloat16") from None


def _ptr(t: Optional[torch.Tensor], name: str, dtype: Optional[torch.dtype] = None) -> Optional[int]:
    if t is None:
        return None
    if not t.is_cuda:
        raise RavenHipError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")
    if not t.is_contiguous():
        raise RavenHipError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise RavenHipError(f"{name} has dtype {t.dtype}, expected {dtype}")
    return t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def make_dims(n_embd: int, n_heads: int, intermediate: int, eps: float, dtype: torch.dtype) -> Dims:
    return Dims(n_embd, n_heads, n_embd // n_heads, intermediate, eps, dtype_code(dtype))


def make_cache(k: torch.Tensor, v: torch.Tensor, steps_present: Optional[torch.Tensor] = None, lookup_mode: int = LOOKUP_NONE,
               core_slot0: int = 0) -> KVCache:
    """k, v: [n_slots, batch, nh, t_max, hd], contiguous, on the GPU; steps_present: int32 [t_max] or None."""
    if k.shape != v.shape or k.dim() != 5:
        raise RavenHipError("cache tensors must be [n_slots, batch, nh, t_max, hd] and of equal shape")
    if steps_present is not None and (steps_present.dtype != torch.int32 or steps_present.numel() < k.shape[3]):
        raise RavenHipError("steps_present must be int32 with one entry per cache position")
    return KVCache(_ptr(k, "cache.k"), _ptr(v, "cache.v", k.dtype), k.shape[0], k.shape[1], k.shape[3], int(lookup_mode),
                   _ptr(steps_present, "steps_present", torch.int32), int(core_slot0))


def make_block_weights(norm_1, norm_2, norm_3, norm_4, wqkv, qk_bias, proj, fc, mlp_proj) -> BlockWeights:
    dt = wqkv.dtype
    return BlockWeights(_ptr(norm_1, "norm_1", dt), _ptr(norm_2, "norm_2", dt), _ptr(norm_3, "norm_3", dt),
                        _ptr(norm_4, "norm_4", dt), _ptr(wqkv, "wqkv", dt), _ptr(qk_bias, "qk_bias", dt),
                        _ptr(proj, "proj", dt), _ptr(fc, "fc", dt), _ptr(mlp_proj, "mlp_proj", dt))


# ---------------------------------------------------------------------------------------------
# per-kernel wrappers (used by the tests and by the host model)
# ---------------------------------------------------------------------------------------------
def rmsnorm_residual(x, weight, eps, residual=None, weight2=None, want_sum=False, want_y=True):
    """Returns (y, sum, y2); entries not asked for are None.  x: [..., dim]."""
    dt = x.dtype
    dim = x.shape[-1]
    rows = x.numel() // dim
    y = torch.empty_like(x) if want_y else None
    s = torch.empty_like(x) if (want_sum and residual is not None) else None
    y2 = torch.empty_like(x) if weight2 is not None else None
    rc = load().raven_rmsnorm_residual(_ptr(x, "x"), _ptr(residual, "residual", dt), _ptr(weight, "weight", dt),
                                       _ptr(y, "y"), _ptr(s, "sum"), _ptr(weight2, "weight2", dt), _ptr(y2, "y2"),
                                       rows, dim, eps, dtype_code(dt), _stream())
    _check(rc, "raven_rmsnorm_residual")
    return y, s, y2


def gemm(x, w, residual=None, out_f32=False):
    """x [M, K], w [N, K] -> [M, N]."""
    dt = x.dtype
    M, K = x.shape
    N = w.shape[0]
    assert w.shape[1] == K
    y = torch.empty(M, N, device=x.device, dtype=torch.float32 if out_f32 else dt)
    rc = load().raven_gemm(_ptr(x, "x"), _ptr(w, "w", dt), _ptr(residual, "residual", dt), _ptr(y, "y"),
                           M, N, K, dtype_code(dt), int(out_f32), _stream())
    _check(rc, "raven_gemm")
    return y


def adapter_gemm_concat(x0, x1, w):
    dt = x0.dtype
    M, K0 = x0.shape
    K1 = x1.shape[1]
    N = w.shape[0]
    assert w.shape[1] == K0 + K1 and x1.shape[0] == M
    y = torch.empty(M, N, device=x0.device, dtype=dt)
    rc = load().raven_adapter_gemm_concat(_ptr(x0, "x0"), _ptr(x1, "x1", dt), _ptr(w, "w", dt), _ptr(y, "y"),
                                          M, N, K0, K1, dtype_code(dt), _stream())
    _check(rc, "raven_adapter_gemm_concat")
    return y


def gemm_swiglu(x, fc):
    dt = x.dtype
    M, K = x.shape
    inter = fc.shape[0] // 2
    assert fc.shape[1] == K
    y = torch.empty(M, inter, device=x.device, dtype=dt)
    rc = load().raven_gemm_swiglu(_ptr(x, "x"), _ptr(fc, "fc", dt), _ptr(y, "out"), M, inter, K, dtype_code(dt), _stream())
    _check(rc, "raven_gemm_swiglu")
    return y


def register_packed_weight(w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Line-aligned copy of a bf16 weight matrix [rows, K] for the tiled GEMM; returns the copy, which the caller keeps
    alive (together with w) until unregister_packed_weight(w).  `out`: a buffer of an earlier registration of the same
    shape to fill again (its address may be held by captured graphs)."""
    assert w.dim() == 2 and w.dtype == torch.bfloat16 and w.is_contiguous()
    rows, K = w.shape
    n = load().raven_packed_weight_bytes(rows, K)
    packed = out if out is not None else torch.empty(n, dtype=torch.uint8, device=w.device)
    assert packed.numel() == n and packed.dtype == torch.uint8 and packed.device == w.device
    rc = load().raven_register_packed_weight(_ptr(w, "w"), rows, K, _ptr(packed, "packed"), _stream())
    _check(rc, "raven_register_packed_weight")
    return packed


def unregister_packed_weight(w: torch.Tensor) -> None:
    _check(load().raven_unregister_packed_weight(_ptr(w, "w")), "raven_unregister_packed_weight")


def linear_workspace(M, n_out_max, device):
    n = load().raven_linear_workspace_bytes(M, n_out_max)
    return torch.empty(max(n, 256), dtype=torch.uint8, device=device)


def linear(x0, w, x1=None, residual=None, swiglu=False, out_f32=False, workspace=None):
    """concat(x0, x1) W^T with the plain / residual / float / SwiGLU epilogues; x0 [M, K0], w [N or 2N, K0 + K1]."""
    dt = x0.dtype
    M, K0 = x0.shape
    K1 = 0 if x1 is None else x1.shape[1]
    N = w.shape[0] // 2 if swiglu else w.shape[0]
    assert w.shape[1] == K0 + K1
    y = torch.empty(M, N, device=x0.device, dtype=torch.float32 if out_f32 else dt)
    rc = load().raven_linear(_ptr(x0, "x0"), _ptr(x1, "x1", dt), _ptr(w, "w", dt), _ptr(residual, "residual", dt), _ptr(y, "y"),
                             M, N, K0, K1, int(swiglu), int(out_f32), dtype_code(dt), _ptr(workspace, "workspace", torch.uint8),
                             0 if workspace is None else workspace.numel(), _stream())
    _check(rc, "raven_linear")
    return y


def paged_kv_append(k, v, k_cache, v_cache, slot_mapping, layout: int = PAGED_NHD):
    """k, v [T, nh * hd] -> k_cache / v_cache (layout NHD: [num_blocks, block_size, nh, hd], HND: [num_blocks, nh, block_size, hd])
    at the flat slots slot_mapping [T] (int64, block * block_size + offset)."""
    T = k.shape[0]
    bs, nh, hd = _paged_dims(k_cache, layout)
    rc = load().raven_paged_kv_append(_ptr(k, "k"), _ptr(v, "v", k.dtype), _ptr(k_cache, "k_cache", k.dtype), _ptr(v_cache, "v_cache", k.dtype),
                                      _ptr(slot_mapping, "slot_mapping", torch.int64), T, nh, hd, bs, layout, dtype_code(k.dtype), _stream())
    _check(rc, "raven_paged_kv_append")


def paged_qkv_rope_append(qkv, qk_bias, freqs, positions, slot_mapping, k_cache, v_cache, layout: int = PAGED_NHD):
    """Rows qkv [T, 3 * nh * hd] of any sequences: bias and rotation of positions [T] (int64) on q and k; returns q [T, nh * hd]
    and writes k, v to the flat slots slot_mapping [T] (int64) of the pages."""
    T = qkv.shape[0]
    bs, nh, hd = _paged_dims(k_cache, layout)
    if qkv.shape[1] != 3 * nh * hd or positions.shape != (T,) or slot_mapping.shape != (T,):
        raise RavenHipError("paged_qkv_rope_append: qkv [T, 3 * nh * hd], positions [T] and slot_mapping [T] do not fit together")
    q = torch.empty(T, nh * hd, device=qkv.device, dtype=qkv.dtype)
    rc = load().raven_paged_qkv_rope_append(
        _ptr(qkv, "qkv"), _ptr(qk_bias, "qk_bias", qkv.dtype), _ptr(freqs, "freqs", torch.float32), _ptr(positions, "positions", torch.int64),
        _ptr(slot_mapping, "slot_mapping", torch.int64), _ptr(q, "q"), _ptr(k_cache, "k_cache", qkv.dtype), _ptr(v_cache, "v_cache", qkv.dtype),
        T, nh, hd, bs, layout, dtype_code(qkv.dtype), _stream())
    _check(rc, "raven_paged_qkv_rope_append")
    return q


def paged_prefill_attention(q, k_cache, v_cache, block_table, seq_lens, q_start, max_q_len: int, layout: int = PAGED_NHD):
    """Causal attention of the rows q [T, nh * hd] (bf16) of several sequences over their pages: sequence b owns rows
    q_start[b] .. q_start[b + 1] - 1 (q_start [B + 1] int32), the last positions of its seq_lens[b] cached ones."""
    B = seq_lens.shape[0]
    if q_start.shape != (B + 1,) or block_table.dim() != 2 or block_table.shape[0] != B:
        raise RavenHipError("paged_prefill_attention: block_table [B, max_blocks], seq_lens [B] and q_start [B + 1] do not fit together")
    block_size, nh, hd = _paged_dims(k_cache, layout)
    y = torch.empty_like(q)
    rc = load().raven_paged_prefill_attention(
        _ptr(q, "q"), _ptr(y, "y"), _ptr(k_cache, "k_cache", q.dtype), _ptr(v_cache, "v_cache", q.dtype),
        _ptr(block_table, "block_table", torch.int32), _ptr(seq_lens, "seq_lens", torch.int32), _ptr(q_start, "q_start", torch.int32),
        B, int(max_q_len), block_table.shape[1], block_size, layout, nh, hd, dtype_code(q.dtype), _stream())
    _check(rc, "raven_paged_prefill_attention")
    return y


def paged_decode_attention(q, k_cache, v_cache, block_table, seq_lens, max_seq_len, workspace=None, layout: int = PAGED_NHD):
    """q [B, nh * hd]; k_cache / v_cache as in paged_kv_append; block_table [B, max_blocks] int32; seq_lens [B] int32."""
    B = q.shape[0]
    block_size, nh, hd = _paged_dims(k_cache, layout)
    y = torch.empty_like(q)
    rc = load().raven_paged_decode_attention(
        _ptr(q, "q"), _ptr(y, "y"), _ptr(k_cache, "k_cache", q.dtype), _ptr(v_cache, "v_cache", q.dtype),
        _ptr(block_table, "block_table", torch.int32), _ptr(seq_lens, "seq_lens", torch.int32), B, block_table.shape[1], block_size,
        layout, int(max_seq_len), nh, hd, dtype_code(q.dtype), _ptr(workspace, "workspace", torch.uint8),
        0 if workspace is None else workspace.numel(), _stream())
    _check(rc, "raven_paged_decode_attention")
    return y


def paged_qkv_attention_decode(qkv, qk_bias, freqs, k_cache, v_cache, block_table, seq_lens, max_seq_len, workspace=None,
                               layout: int = PAGED_NHD):
    """The decode step of a paged attention layer in one launch: qkv [B, 3 * nh * hd] from the fused projection; bias, RoPE at
    position seq_lens[b] - 1, write of the new k / v row to its page, attention over seq_lens[b] positions.  Returns y [B, nh * hd]."""
    B = qkv.shape[0]
    block_size, nh, hd = _paged_dims(k_cache, layout)
    y = torch.empty(B, nh * hd, device=qkv.device, dtype=qkv.dtype)
    rc = load().raven_paged_qkv_attention_decode(
        _ptr(qkv, "qkv"), _ptr(qk_bias, "qk_bias", qkv.dtype), _ptr(freqs, "freqs", torch.float32), _ptr(y, "y"),
        _ptr(k_cache, "k_cache", qkv.dtype), _ptr(v_cache, "v_cache", qkv.dtype), _ptr(block_table, "block_table", torch.int32),
        _ptr(seq_lens, "seq_lens", torch.int32), B, block_table.shape[1], block_size, layout, int(max_seq_len), nh, hd, dtype_code(qkv.dtype),
        _ptr(workspace, "workspace", torch.uint8), 0 if workspace is None else workspace.numel(), _stream())
    _check(rc, "raven_paged_qkv_attention_decode")
    return y


EXIT_ENTROPY, EXIT_KL, EXIT_MINP_KL = 0, 1, 2


def exit_logit_stats(logits, kind: int, prev_log_probs=None):
    """One float per row of logits [rows, V] (float): entropy, or KL against prev_log_probs, which is overwritten."""
    rows, V = logits.shape
    out = torch.empty(rows, device=logits.device, dtype=torch.float32)
    rc = load().raven_exit_logit_stats(_ptr(logits, "logits", torch.float32), _ptr(prev_log_probs, "prev_log_probs", torch.float32),
                                       _ptr(out, "out"), rows, V, int(kind), _stream())
    _check(rc, "raven_exit_logit_stats")
    return out


def exit_latent_stats(latents, prev, want_rel=True, want_cos=False):
    """latents, prev [rows, h] -> (|latents - prev| / |latents|, cosine), each [rows] in the inputs' dtype or None."""
    rows, h = latents.shape
    rel = torch.empty(rows, device=latents.device, dtype=latents.dtype) if want_rel else None
    cos = torch.empty(rows, device=latents.device, dtype=latents.dtype) if want_cos else None
    rc = load().raven_exit_latent_stats(_ptr(latents, "latents"), _ptr(prev, "prev", latents.dtype), _ptr(rel, "rel"), _ptr(cos, "cos"),
                                        rows, h, dtype_code(latents.dtype), _stream())
    _check(rc, "raven_exit_latent_stats")
    return rel, cos


def gemv_fused(x0, w, x1=None, norm_a=None, norm_b=None, want_xa=False, residual=None, swiglu=False, out_f32=False, eps=1e-6):
    """One token row: (norms on x0) -> concat(x0, x1) W^T -> epilogue.  Returns (y, norm_a(x0) or None)."""
    dt = x0.dtype
    K0 = x0.numel()
    K1 = 0 if x1 is None else x1.numel()
    N = w.shape[0] // 2 if swiglu else w.shape[0]
    assert w.shape[1] == K0 + K1
    y = torch.empty(N, device=x0.device, dtype=torch.float32 if out_f32 else dt)
    xa = torch.empty_like(x0) if want_xa else None
    rc = load().raven_gemv_fused(_ptr(x0, "x0"), _ptr(x1, "x1", dt), _ptr(norm_a, "norm_a", dt), _ptr(norm_b, "norm_b", dt),
                                 _ptr(xa, "xa_out"), _ptr(w, "w", dt), _ptr(residual, "residual", dt), _ptr(y, "y"), N, K0, K1,
                                 eps, int(swiglu), int(out_f32), dtype_code(dt), _stream())
    _check(rc, "raven_gemv_fused")
    return y, xa


def qkv_bias_rope_cache_append(qkv, qk_bias, freqs, cache: KVCache, slot, B, S, pos0, n_heads, head_dim, pos_dev=None):
    dt = qkv.dtype
    q = torch.empty(B * S, n_heads * head_dim, device=qkv.device, dtype=dt)
    rc = load().raven_qkv_bias_rope_cache_append(
        _ptr(qkv, "qkv"), _ptr(qk_bias, "qk_bias", dt), _ptr(freqs, "freqs", torch.float32), _ptr(q, "q"),
        C.byref(cache), slot, B, S, pos0, _ptr(pos_dev, "pos_dev", torch.int32), n_heads, head_dim, dtype_code(dt), _stream())
    _check(rc, "raven_qkv_bias_rope_cache_append")
    return q


def attention_workspace(M, n_heads, head_dim, device):
    """Scratch for split partials (None when the shape never splits)."""
    n = load().raven_decode_attention_workspace_bytes(M, n_heads, head_dim)
    return torch.empty(n, dtype=torch.uint8, device=device) if n else None


def decode_attention(q, cache: KVCache, slot, B, S, pos0, n_heads, head_dim, pos_dev=None, workspace=None):
    y = torch.empty_like(q)
    rc = load().raven_decode_attention(
        _ptr(q, "q"), _ptr(y, "y"), C.byref(cache), slot, B, S, pos0, _ptr(pos_dev, "pos_dev", torch.int32),
        n_heads, head_dim, dtype_code(q.dtype), _ptr(workspace, "workspace", torch.uint8),
        0 if workspace is None else workspace.numel(), _stream())
    _check(rc, "raven_decode_attention")
    return y


def qkv_attention_decode(qkv, qk_bias, freqs, cache: KVCache, slot, B, pos0, n_heads, head_dim, pos_dev=None, workspace=None):
    """Decode step: fused qkv rows [B, 3h] -> attention output [B, h]; appends k, v at pos0."""
    dt = qkv.dtype
    y = torch.empty(B, n_heads * head_dim, device=qkv.device, dtype=dt)
    rc = load().raven_qkv_attention_decode(
        _ptr(qkv, "qkv"), _ptr(qk_bias, "qk_bias", dt), _ptr(freqs, "freqs", torch.float32), _ptr(y, "y"), C.byref(cache),
        slot, B, pos0, _ptr(pos_dev, "pos_dev", torch.int32), n_heads, head_dim, dtype_code(dt),
        _ptr(workspace, "workspace", torch.uint8), 0 if workspace is None else workspace.numel(), _stream())
    _check(rc, "raven_qkv_attention_decode")
    return y


def qkv_attention_decode_static(qkv, qk_bias, freqs, cache: KVCache, slot, B, pos0, n_heads, head_dim, pos_dev=None, out=None):
    """The decode step of qkv_attention_decode without a workspace: partial results go to the library's built-in buffer.
    With `out` given nothing is allocated on the way (for callers that cannot allocate)."""
    dt = qkv.dtype
    y = out if out is not None else torch.empty(B, n_heads * head_dim, device=qkv.device, dtype=dt)
    rc = load().raven_qkv_attention_decode_static(
        _ptr(qkv, "qkv"), _ptr(qk_bias, "qk_bias", dt), _ptr(freqs, "freqs", torch.float32), _ptr(y, "y", dt), C.byref(cache),
        slot, B, pos0, _ptr(pos_dev, "pos_dev", torch.int32), n_heads, head_dim, dtype_code(dt), _stream())
    _check(rc, "raven_qkv_attention_decode_static")
    return y


def prefill_attention(q, cache: KVCache, slot, B, S, pos0, n_heads, head_dim, pos_dev=None):
    y = torch.empty_like(q)
    rc = load().raven_prefill_attention(
        _ptr(q, "q"), _ptr(y, "y"), C.byref(cache), slot, B, S, pos0, _ptr(pos_dev, "pos_dev", torch.int32),
        n_heads, head_dim, dtype_code(q.dtype), _stream())
    _check(rc, "raven_prefill_attention")
    return y


def swiglu(z):
    """z [M, 2I] -> [M, I]."""
    M, two_i = z.shape
    out = torch.empty(M, two_i // 2, device=z.device, dtype=z.dtype)
    _check(load().raven_swiglu(_ptr(z, "z"), _ptr(out, "out"), M, two_i // 2, dtype_code(z.dtype), _stream()), "raven_swiglu")
    return out


def noise_mix(x, noise, keep: float, a: float, d: float = 0.0):
    """T(T(x * keep) + T(noise * a) [/ d, rounded again]) elementwise; x and noise of one shape and dtype."""
    if noise.shape != x.shape:
        raise RavenHipError(f"noise_mix: noise {tuple(noise.shape)} against x {tuple(x.shape)}")
    y = torch.empty_like(x)
    rc = load().raven_noise_mix(_ptr(x, "x"), _ptr(noise, "noise", x.dtype), _ptr(y, "y"), x.numel(), float(keep), float(a), float(d),
                                dtype_code(x.dtype), _stream())
    _check(rc, "raven_noise_mix")
    return y


def embed(wte, ids, scale, out=None):
    M = ids.numel()
    dim = wte.shape[1]
    if out is None:
        out = torch.empty(M, dim, device=wte.device, dtype=wte.dtype)
    rc = load().raven_embed(_ptr(wte, "wte"), _ptr(ids, "ids", torch.int64), _ptr(out, "out", wte.dtype), M, dim,
                            wte.shape[0], scale, dtype_code(wte.dtype), _stream())
    _check(rc, "raven_embed")
    return out


def argmax(logits, out=None):
    M, V = logits.shape
    if out is None:
        out = torch.empty(M, device=logits.device, dtype=torch.int64)
    rc = load().raven_argmax(_ptr(logits, "logits", torch.float32), _ptr(out, "out", torch.int64), M, V, _stream())
    _check(rc, "raven_argmax")
    return out


def advance_pos(pos_dev, delta=1):
    _check(load().raven_advance_pos(_ptr(pos_dev, "pos_dev", torch.int32), delta, _stream()), "raven_advance_pos")


def block_workspace(dims: Dims, M: int, device) -> torch.Tensor:
    n = load().raven_block_workspace_bytes(C.byref(dims), M)
    return torch.zeros(max(n, 256), dtype=torch.uint8, device=device)


def sandwich_block(dims: Dims, w: BlockWeights, x_in, x_out, freqs, cache: KVCache, slot, B, S, pos0, workspace,
                   ln_f=None, pos_dev=None):
    rc = load().raven_sandwich_block(
        C.byref(dims), C.byref(w), _ptr(ln_f, "ln_f", x_in.dtype), _ptr(x_in, "x_in"), _ptr(x_out, "x_out", x_in.dtype),
        _ptr(freqs, "freqs", torch.float32), C.byref(cache), slot, B, S, pos0, _ptr(pos_dev, "pos_dev", torch.int32),
        _ptr(workspace, "workspace", torch.uint8), workspace.numel(), _stream())
    _check(rc, "raven_sandwich_block")
    return x_out


def core_iteration(dims: Dims, adapter_w, blocks, state_in, embeds, state_out, freqs, cache: KVCache, first_slot,
                   B, S, pos0, workspace, ln_f=None, pos_dev=None):
    """blocks: a ctypes array (BlockWeights * n)."""
    rc = load().raven_core_iteration(
        C.byref(dims), _ptr(adapter_w, "adapter_w", state_in.dtype), blocks, len(blocks), _ptr(ln_f, "ln_f", state_in.dtype),
        _ptr(state_in, "state_in"), _ptr(embeds, "embeds", state_in.dtype), _ptr(state_out, "state_out", state_in.dtype),
        _ptr(freqs, "freqs", torch.float32), C.byref(cache), first_slot, B, S, pos0,
        _ptr(pos_dev, "pos_dev", torch.int32), _ptr(workspace, "workspace", torch.uint8), workspace.numel(), _stream())
    _check(rc, "raven_core_iteration")
    return state_out


def core_iterations(dims: Dims, adapter_w, blocks, state_in, embeds, state_out, freqs, cache: KVCache, slots, B, S, pos0,
                    workspace, ln_f=None, pos_dev=None):
    """slots: one list of len(blocks) cache slots per recurrence; runs len(slots) recurrences."""
    flat = [int(v) for it in slots for v in it]
    if len(flat) != len(slots) * len(blocks):
        raise RavenHipError("core_iterations: every recurrence needs one slot per block")
    arr = (C.c_int32 * len(flat))(*flat)
    rc = load().raven_core_iterations(
        C.byref(dims), _ptr(adapter_w, "adapter_w", state_in.dtype), blocks, len(blocks), _ptr(ln_f, "ln_f", state_in.dtype),
        _ptr(state_in, "state_in"), _ptr(embeds, "embeds", state_in.dtype), _ptr(state_out, "state_out", state_in.dtype),
        _ptr(freqs, "freqs", torch.float32), C.byref(cache), arr, len(slots), B, S, pos0,
        _ptr(pos_dev, "pos_dev", torch.int32), _ptr(workspace, "workspace", torch.uint8), workspace.numel(), _stream())
    _check(rc, "raven_core_iterations")
    return state_out


def make_paged_kv(k_caches, v_caches, block_table, seq_lens, max_seq_len: int, layout: int = PAGED_NHD) -> PagedKV:
    """k_caches / v_caches: one paged cache tensor (as in paged_kv_append) per block of the stack; block_table [B, max_blocks] and
    seq_lens [B] int32 on the GPU.  The returned structure holds pointers only: keep the tensors alive."""
    if len(k_caches) != len(v_caches) or not k_caches:
        raise RavenHipError("make_paged_kv: one key and one value cache per block")
    shape, dt = k_caches[0].shape, k_caches[0].dtype
    for t in list(k_caches) + list(v_caches):
        if t.shape != shape or t.dtype != dt:
            raise RavenHipError("make_paged_kv: all caches must share shape and dtype")
    ka = (C.c_void_p * len(k_caches))(*[_ptr(t, "k_cache") for t in k_caches])
    va = (C.c_void_p * len(v_caches))(*[_ptr(t, "v_cache") for t in v_caches])
    if block_table.dim() != 2 or seq_lens.shape != (block_table.shape[0],):
        raise RavenHipError("make_paged_kv: block_table [B, max_blocks], seq_lens [B]")
    kv = PagedKV(C.cast(ka, C.POINTER(C.c_void_p)), C.cast(va, C.POINTER(C.c_void_p)), _ptr(block_table, "block_table", torch.int32),
                 _ptr(seq_lens, "seq_lens", torch.int32), block_table.shape[1], _paged_dims(k_caches[0], layout)[0], int(max_seq_len), layout)
    kv._keep = (ka, va)  # the pointer arrays live in host memory owned by this object
    return kv


def paged_decode_blocks(dims: Dims, blocks, x_in, x_out, freqs, kv: PagedKV, B, workspace, adapter_w=None, embeds=None, n_iterations=1,
                        ln_f=None):
    """The blocks once (adapter_w None: prelude, coda) or n_iterations x (adapter([x, embeds]) + blocks) over paged caches."""
    rc = load().raven_paged_decode_blocks(
        C.byref(dims), _ptr(adapter_w, "adapter_w", x_in.dtype), blocks, len(blocks), _ptr(ln_f, "ln_f", x_in.dtype), _ptr(x_in, "x_in"),
        _ptr(embeds, "embeds", x_in.dtype), _ptr(x_out, "x_out", x_in.dtype), _ptr(freqs, "freqs", torch.float32), C.byref(kv),
        int(n_iterations), B, _ptr(workspace, "workspace", torch.uint8), workspace.numel(), _stream())
    _check(rc, "raven_paged_decode_blocks")
    return x_out
