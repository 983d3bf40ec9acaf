"""Python bindings of the HIP kernels: each function checks on the host that the
operands have the shapes, element types, layout and device that the kernel and
its grid assume, then launches on the current HIP stream.

There is no fallback: if the library cannot be built or loaded, or no GPU is
present, importing the kernels fails with the reason.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import build as _build

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}

ALGO_AUTO, ALGO_GENERIC, ALGO_FAST = 0, 1, 2
ALGO_TILE = 1000   # ALGO_TILE + 256, 128 or 64: the tiled MFMA gemm with tiles of that many rows (+ 512: 256 x 256; + 65: 64 rows, k step 128)
EPI_STORE, EPI_RESIDUAL, EPI_SILU_MUL, EPI_PARTIAL, EPI_SILU_MUL_IL = 0, 1, 2, 3, 4
DECODE_SPLIT_KEYS = 128   # keys per split of the decode attention kernel


class KernelError(RuntimeError):
    pass


_lib = None


def load_library():
    """Load (building first if need be) the kernel library.  Raises if there is no GPU."""
    global _lib
    if _lib is not None:
        return _lib
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible: the engine has no CPU path")
    path = _build.library_path()
    lib = ctypes.CDLL(str(path))
    lib.qe_last_error.restype = ctypes.c_char_p
    vp, i32, f32, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_long
    sigs = {
        "qe_embedding": [vp, vp, vp, i32, i32, i32, i32, vp],
        "qe_rmsnorm": [vp, vp, i32, i32, i64, vp, vp, vp, i32, i32, f32, i32, i32, vp],
        "qe_residual_add": [vp, vp, i64, i32, vp],
        "qe_scatter_int": [vp, vp, vp, i32, i64, vp],
        "qe_silu_mul": [vp, vp, i32, i32, i32, i32, vp],
        "qe_gemm_silu_supported": [i32, i32, i32, i32, i32],
        "qe_gemm": [vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, i32, i32, vp, f32, vp, i32, vp, vp],
        "qe_gemm_norm_supported": [i32, i32, i32, i32],
        "qe_gemm_norm_preferred": [i32, i32, i32, i32, i32],
        "qe_gemm_norm_max_rows": [],
        "qe_gemm_partial_splits": [i32, i32, i32],
        "qe_gemm_qkv_supported": [i32, i32, i32, i32, i32, i32, i32, i32],
        "qe_gemm_qkv_run": [vp, vp, vp, i32, i32, i32, i32, i32, vp, vp, vp, vp, f32, vp, vp, vp, i32, vp],
        "qe_gemm_fused_supported": [i32, i32, i32, i32, i32],
        "qe_attention_decode_supported": [i32, i32, i32, i32, i32],
        "qe_attention_prefill_supported": [i32, i32, i32, i32, i32],
        "qe_attention_prefill_rows": [i32, i32],
        "qe_attention_prefill_run": [vp, vp, vp, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, f32, i32, i32, i32, i32, i32, i32,
                                     i32, vp, i64, vp],
        "qe_attention_prefill_plan_segments": [i32, i32, i32],
        "qe_attention_prefill_tiles_run": [vp, i32, i32, vp, i32, vp],
        "qe_attention_prefill_workspace_bytes_for": [i32, i32, i32, i32, i32],
        "qe_attention_prefill_plan": [i32, i32, i32, i32],
        "qe_attention_prefill_plan_uncut_keys": [],
        "qe_attention_prefill_workspace_bytes": [i32, i32, i32, i32, i32, i32],
        "qe_attention_decode_run": [vp, vp, vp, vp, i32, vp, vp, vp, i32, vp, i32, i32, i32, i32, f32, i32, i32, i32, i32, i32, vp, i64, vp],
        "qe_attention_decode_fused_run": [vp, vp, vp, vp, i32, vp, vp, vp, i32, vp, vp, vp, vp, f32, vp,
                                          i32, i32, i32, i32, f32, i32, i32, i32, vp, i64, vp],
        "qe_qk_rope_store": [vp, vp, vp, vp, f32, vp, i32, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp],
        "qe_qk_rope_store_parts": [vp, i32, vp, vp, vp, vp, f32, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, vp],
        "qe_qk_rope_store_parts_supported": [i32, i32],
        "qe_gemm_partial_preferred": [i32, i32, i32, i32, i32],
        "qe_gemm_branch_splits": [i32, i32, i32, i32, i32],
        "qe_attention": [vp, vp, vp, vp, vp, vp, i32, vp, i32, i32, i32, i32, i32, f32, i32, i32, i32, i32, vp],
        "qe_qkv_conv_rope_store": [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, i32, i32, i32, i32, vp],
        "qe_scale_f32": [vp, i64, f32, vp],
        "qe_moe_route_biased": [vp, vp, vp, vp, i32, i32, i32, f32, i32, vp, i32, vp],
        "qe_moe_front_small_supported": [i32, i32, i32],
        "qe_moe_front_small": [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, i32, i32, vp, i32, vp],
        "qe_moe_row_gate": [vp, vp, i32, vp, i64, i32, i32, i32, vp],
        "qe_diff_heads": [vp, vp, vp, i64, i32, i32, i32, i32, i32, f32, f32, f32, i32, vp],
        "qe_moe_identity": [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp],
        "qe_argmax": [vp, vp, i32, i32, vp, i64, vp],
        "qe_argmax_static": [vp, vp, i32, i32, vp],
        "qe_sample": [vp, vp, vp, vp, i32, i32, vp],
        "qe_postnorm": [vp, vp, i32, i32, f32, vp, i32, f32, vp, i32, i32, i32, vp],
        "qe_qkv_norm_store": [vp, i32, vp, vp, i32, f32, i32, i32, f32, vp, vp, i32, vp, vp, i32, vp, vp, vp,
                              i32, i32, i32, i32, i32, i32, i32, i32, i32, vp],
        "qe_attention_talk": [vp, vp, i64, f32, vp, vp, vp, vp, i32, vp, i32, vp, i32, vp, i32, i32, i32, i32, i32, i32,
                              f32, i32, i32, vp, i32, vp],
        "qe_attention_talk_splits": [i32, i32],
        "qe_token_shift": [vp, vp, i32, vp, i64, vp, vp, i32, i32, i32, i32, vp],
        "qe_recurrence_chunk_len": [i32],
        "qe_linear_recurrence_chunked": [vp, vp, vp, i64, vp, i64, vp, vp, vp, i32, i32, vp, i64, vp, vp, i32, vp, i32, vp, vp,
                                         i32, i32, i32, i32, vp],
        "qe_linear_recurrence": [vp, vp, vp, i64, vp, i64, vp, vp, vp, i32, i32, vp, i64, vp, vp, i32, i32, i32, i32,
                                 i32, vp],
        "qe_gated_norm": [vp, vp, vp, i64, i32, i32, f32, f32, vp, i64, i32, i32, i32, i32, vp],
        "qe_unary": [vp, i32, vp, i32, i64, i32, f32, vp],
        "qe_scaled_sum": [vp, f32, vp, f32, i32, vp, i64, vp],
        "qe_polynorm": [vp, vp, f32, vp, i32, i32, i32, vp],
        "qe_short_conv": [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp],
        "qe_latent_kv_store": [vp, vp, f32, vp, vp, i32, vp, vp, i32, i32, i32, i32, vp, vp, i32, i32, i32, vp],
        "qe_latent_q_rotate": [vp, vp, vp, i32, vp, i32, i32, i32, i32, i32, i32, i32, vp],
        "qe_latent_attention": [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, i32, vp, i32, vp],
        "qe_latent_attention_mfma_supported": [i32, i32],
        "qe_latent_attention_mfma": [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, i32, vp, vp, i64, vp],
        "qe_gemm_heads": [vp, i64, i64, vp, vp, i64, i64, vp, i64, i64, i64, i32, i32, i32, i32, i32, i32, vp],
        "qe_gemm_heads_mfma_supported": [i32, i64, i64],
        "qe_gemm_heads_mfma": [vp, i64, i64, vp, vp, i64, i64, vp, i64, i64, i64, i32, i32, i32, i32, vp],
        "qe_moe_route": [vp, vp, vp, i32, i32, i32, i32, i32, vp],
        "qe_moe_sort": [vp, i32, i32, i32, i32, vp, vp, vp, vp, i32, vp],
        "qe_moe_gemm": [vp, vp, i32, vp, vp, vp, vp, vp, i32, i32, i32, i32, f32, f32, i32, i32, i32, i32, vp],
        "qe_moe_gather": [vp, vp, i32, vp, i32, i32, i32, vp],
        "qe_moe_combine": [vp, vp, vp, vp, i32, i32, i32, i32, vp],
        "qe_gemm_mfma_grouped": [vp, vp, vp, vp, vp, i32, i32, i32, i32, f32, f32, i32, vp],
        "qe_gemm_mfma_grouped_tile_rows": [],
        "qe_moe_tile_rows": [],
        "qe_moe_gemm_mfma_supported": [i32],
        "qe_moe_gemm_mfma": [vp, vp, i32, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, f32, f32, i32, i32, vp],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = ctypes.c_int
    lib.qe_use_matrix_f32.argtypes = [i32]
    lib.qe_use_matrix_f32.restype = None
    lib.qe_mfma_probe.argtypes = [vp, i32, i32, ctypes.POINTER(ctypes.c_double), vp]
    lib.qe_mfma_probe.restype = ctypes.c_int
    lib.qe_argmax_workspace_bytes.argtypes = [i32, i32]
    lib.qe_argmax_workspace_bytes.restype = ctypes.c_long
    lib.qe_argmax_static_max_bytes.argtypes = []
    lib.qe_argmax_static_max_bytes.restype = ctypes.c_long
    lib.qe_attention_decode_workspace_bytes.argtypes = [i32, i32, i32, i32, i32]
    lib.qe_attention_decode_workspace_bytes.restype = ctypes.c_long
    lib.qe_attention_prefill_workspace_bytes.restype = ctypes.c_long
    lib.qe_latent_attention_mfma_workspace_bytes.argtypes = [i32, i32, i32, i32]
    lib.qe_latent_attention_mfma_workspace_bytes.restype = ctypes.c_long
    lib.qe_attention_prefill_workspace_bytes_for.restype = ctypes.c_long
    _lib = lib
    return lib


def library_file() -> str:
    load_library()
    return str(_build.library_path(verbose=False))


_fixed_stream: Optional[int] = None


def _stream() -> int:
    return _fixed_stream if _fixed_stream is not None else torch.cuda.current_stream().cuda_stream


class one_stream:
    """Within this scope every kernel goes to the stream that is current on entry: asking torch
    for the current stream costs several microseconds a call, and a step of the model makes a
    few hundred calls on one stream.  (Entered inside whatever stream or graph-capture context the
    caller has set up; scopes nest.)"""

    def __enter__(self):
        global _fixed_stream
        self._outer = _fixed_stream
        _fixed_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _fixed_stream
        _fixed_stream = self._outer
        return False


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = _lib.qe_last_error().decode(errors="replace")
        raise KernelError(f"{what}: {msg} (code {rc})")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need(t: torch.Tensor, name: str, dtype=None, shape=None, device=None) -> None:
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name} is no tensor")
    if not t.is_cuda:
        raise KernelError(f"{name} is not on the GPU")
    if device is not None and t.device != device:
        raise KernelError(f"{name} is on {t.device}, expected {device}")
    if not t.is_contiguous():
        raise KernelError(f"{name} is not contiguous")
    if dtype is not None:
        ok = t.dtype in dtype if isinstance(dtype, (tuple, list)) else t.dtype == dtype
        if not ok:
            raise KernelError(f"{name} has element type {t.dtype}, expected {dtype}")
    if shape is not None:
        if t.dim() != len(shape) or any(s is not None and int(s) != int(a) for s, a in zip(shape, t.shape)):
            raise KernelError(f"{name} has shape {tuple(t.shape)}, expected {tuple(shape)}")


_ACT = (torch.float32, torch.bfloat16)


def embedding(ids: torch.Tensor, table: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = float32(table[ids[t]]).  ids int32 [T] with 0 <= id < V (the caller checks the range)."""
    lib = load_library()
    _need(ids, "ids", torch.int32, (None,))
    _need(table, "table", _ACT, (None, None), ids.device)
    T, (V, H) = ids.shape[0], table.shape
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=ids.device)
    _need(out, "out", torch.float32, (T, H), ids.device)
    _check(lib.qe_embedding(ids.data_ptr(), table.data_ptr(), out.data_ptr(), T, V, H,
                            _DT[table.dtype], _stream()), "embedding")
    return out


def rmsnorm(h: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
            out: Optional[torch.Tensor] = None, center: bool = False) -> torch.Tensor:
    """RMSNorm of the 32-bit stream h [T, H] into out_dtype; with ``center`` a layer norm without bias:
    (v - mean) * rsqrt(mean of the squared deviations + eps) * weight.

    With ``delta`` the residual sum h + delta is normed; it is written back to h
    unless ``rows`` is given.  delta is [T, H] in out_dtype, or float32 [S, T, H]:
    partial products that are added in the order of S.  With ``rows`` (int32 [R])
    only those rows are normed and the result is [R, H].
    """
    lib = load_library()
    _need(h, "h", torch.float32, (None, None))
    T, H = h.shape
    _need(weight, "weight", torch.float32, (H,), h.device)
    n_delta, dt_d = 0, _DT[out_dtype]
    if delta is not None:
        if delta.dim() == 3:
            _need(delta, "delta", torch.float32, (None, T, H), h.device)
            n_delta, dt_d = delta.shape[0], F32
        else:
            _need(delta, "delta", out_dtype, (T, H), h.device)
            n_delta = 1
    n = T
    if rows is not None:
        _need(rows, "rows", torch.int32, (None,), h.device)
        n = rows.shape[0]
    if out is None:
        out = torch.empty((n, H), dtype=out_dtype, device=h.device)
    _need(out, "out", out_dtype, (n, H), h.device)
    _check(lib.qe_rmsnorm(h.data_ptr(), _ptr(delta), n_delta, dt_d, T, _ptr(rows), weight.data_ptr(),
                          out.data_ptr(), n, H, float(eps), _DT[out_dtype], int(bool(center)), _stream()), "rmsnorm")
    return out


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> None:
    """h += delta, h in 32-bit; delta [T, H], or float32 [S, T, H] partial products added in order."""
    lib = load_library()
    _need(h, "h", torch.float32)
    parts = [delta] if delta.dim() == h.dim() else list(delta.unbind(0))
    for d in parts:
        _need(d, "delta", _ACT, tuple(h.shape), h.device)
        _check(lib.qe_residual_add(h.data_ptr(), d.data_ptr(), h.numel(), _DT[d.dtype], _stream()),
               "residual_add")


def scatter_int(table: torch.Tensor, idx: torch.Tensor, val: torch.Tensor) -> None:
    """table.flatten()[idx[i]] = val[i] wherever idx[i] >= 0 (int32).  The caller guarantees idx < table.numel()."""
    lib = load_library()
    _need(table, "table", torch.int32)
    _need(idx, "idx", torch.int32, (None,), table.device)
    _need(val, "val", torch.int32, (idx.shape[0],), table.device)
    _check(lib.qe_scatter_int(table.data_ptr(), idx.data_ptr(), val.data_ptr(), idx.shape[0], table.numel(),
                              _stream()), "scatter_int")


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """[I, K] gate and up weights -> [2 I, K] with the rows in alternating blocks of 32 (gate 0..31,
    up 0..31, gate 32..63, ...): the layout of EPI_SILU_MUL_IL.  I must be a multiple of 32."""
    I, K = gate.shape
    return torch.stack([gate.view(I // 32, 32, K), up.view(I // 32, 32, K)], dim=1).reshape(2 * I, K).contiguous()


def silu_mul(gu: torch.Tensor, out: Optional[torch.Tensor] = None, interleaved: bool = False) -> torch.Tensor:
    """gu [T, 2 I] = gate | up (or, interleaved, gate and up in alternating blocks of 32)
    ->  silu(gate) * up  [T, I]."""
    lib = load_library()
    _need(gu, "gu", _ACT, (None, None))
    T, I2 = gu.shape
    if I2 % 2:
        raise KernelError(f"silu_mul: the width {I2} of gate|up is odd")
    I = I2 // 2
    if out is None:
        out = torch.empty((T, I), dtype=gu.dtype, device=gu.device)
    _need(out, "out", gu.dtype, (T, I), gu.device)
    _check(lib.qe_silu_mul(gu.data_ptr(), out.data_ptr(), T, I, int(interleaved), _DT[gu.dtype], _stream()),
           "silu_mul")
    return out


def gemm_fused_supported(x: torch.Tensor, w: torch.Tensor) -> bool:
    """True if gemm can add into the residual stream or apply silu-mul itself for these operands."""
    lib = load_library()
    return bool(lib.qe_gemm_fused_supported(x.shape[0], w.shape[0], x.shape[1], _DT[x.dtype], _DT[w.dtype]))


def gemm_silu_supported(x: torch.Tensor, w: torch.Tensor) -> bool:
    """True if gemm can apply silu-mul itself over w = interleaved gate|up rows (EPI_SILU_MUL_IL)."""
    lib = load_library()
    return bool(lib.qe_gemm_silu_supported(x.shape[0], w.shape[0] // 2, x.shape[1], _DT[x.dtype], _DT[w.dtype]))


def gemm_norm_supported(M: int, w: torch.Tensor) -> bool:
    """True if gemm can take the RMSNorm that stands before the product as its prologue (``norm_weight``)
    for M rows of the stream against w: up to 16 rows, bfloat16 weights."""
    lib = load_library()
    return w.dtype in _DT and bool(lib.qe_gemm_norm_supported(int(M), w.shape[0], w.shape[1], _DT[w.dtype]))


def gemm_norm_preferred(M: int, w: torch.Tensor, n_delta: int) -> bool:
    """True if the product of M rows of the stream against w should do the residual sum of ``n_delta``
    partial products and the norm before it in its prologue (gemm with ``norm_weight``) rather than leave
    them to the norm's own kernel: gemm_norm_supported, and the sizes up to which that pays."""
    lib = load_library()
    return w.dtype in _DT and bool(lib.qe_gemm_norm_preferred(int(M), w.shape[0], w.shape[1], _DT[w.dtype], int(n_delta)))


def gemm_norm_max_rows() -> int:
    """No product takes the norm before it as its prologue with more rows than this."""
    return load_library().qe_gemm_norm_max_rows()


def gemm(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
         out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None,
         algo: int = ALGO_AUTO, epilogue: int = EPI_STORE, splits: int = 0,
         norm_weight: Optional[torch.Tensor] = None, norm_eps: float = 0.0,
         delta: Optional[torch.Tensor] = None, stream_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [M, K] . w [N, K]^T (+ bias [N], 32-bit) -> [M, N] in out_dtype (default: x's).

    epilogue EPI_RESIDUAL: the product is added into ``out``, the 32-bit stream [M, N].
    epilogue EPI_SILU_MUL: w is [2 N, K] (gate rows, then up rows); the result is
    silu(x . gate^T) * (x . up^T), [M, N].  EPI_SILU_MUL_IL: the same with the gate and up rows
    interleaved in blocks of 32 (see interleave_gate_up); needs gemm_silu_supported(x, w).
    epilogue EPI_PARTIAL: the product is cut along K into ``splits`` (0: chosen for the shape)
    partial products, returned as float32 [splits, M, N]; their sum over the first index, taken
    in order, is the product.  All three need gemm_fused_supported(x, w).

    norm_weight (float32 [K]) with norm_eps: x is the 32-bit stream and the RMSNorm of its rows, rounded
    to bfloat16 as the norm kernel rounds it, is what is multiplied (out_dtype defaults to bfloat16);
    needs gemm_norm_supported(M, w); with the store and silu-mul epilogues.  With it, ``delta`` (float32
    [S, M, K], the partial products of the branch before) is added to the stream's rows, in the order
    of S, before the norm, and the sums are written to ``stream_out`` [M, K], another tensor than x (every
    block reads x while one of them writes): the residual sum and the norm without kernels of their own."""
    lib = load_library()
    _need(x, "x", _ACT, (None, None))
    M, K = x.shape
    _need(w, "w", _ACT, (None, K), x.device)
    N = w.shape[0]
    if epilogue in (EPI_SILU_MUL, EPI_SILU_MUL_IL):
        if N % 2:
            raise KernelError("gemm: gate|up weights have an odd number of rows")
        N //= 2
    if norm_weight is not None:
        _need(x, "x (the stream)", torch.float32, (M, K))
        _need(norm_weight, "norm_weight", torch.float32, (K,), x.device)
        if not gemm_norm_supported(M, w):
            raise KernelError(f"gemm: {M} rows against {tuple(w.shape)} are not taken with the norm as prologue")
        out_dtype = out_dtype or torch.bfloat16
        if delta is not None:
            _need(delta, "delta", torch.float32, (None, M, K), x.device)
            if stream_out is None:
                raise KernelError("gemm: partial products to add need a place for the summed stream")
            _need(stream_out, "stream_out", torch.float32, (M, K), x.device)
            if stream_out.data_ptr() == x.data_ptr():
                raise KernelError("gemm: the summed stream cannot be written over the stream that is read")
        elif stream_out is not None:
            raise KernelError("gemm: stream_out goes with delta")
    elif delta is not None or stream_out is not None:
        raise KernelError("gemm: delta and stream_out go with norm_weight")
    elif x.dtype == torch.float32 and w.dtype != torch.float32:
        raise KernelError("gemm: 32-bit activations need 32-bit weights")
    if bias is not None:
        _need(bias, "bias", torch.float32, (N,), x.device)
    if epilogue == EPI_RESIDUAL:
        if out is None:
            raise KernelError("gemm: the residual epilogue needs the stream to add into")
        out_dtype = torch.float32
    out_dtype = out_dtype or x.dtype
    shape = (M, N)
    if epilogue == EPI_PARTIAL:
        splits = splits or lib.qe_gemm_partial_splits(M, N, K)
        out_dtype, shape = torch.float32, (splits, M, N)
    else:
        splits = 1
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    _need(out, "out", out_dtype, shape, x.device)
    _check(lib.qe_gemm(x.data_ptr(), w.data_ptr(), _ptr(bias), out.data_ptr(), M, N, K,
                       _DT[x.dtype], _DT[w.dtype], _DT[out_dtype], algo, epilogue, splits,
                       _ptr(norm_weight), float(norm_eps), _ptr(delta), 0 if delta is None else delta.shape[0],
                       _ptr(stream_out), _stream()), "gemm")
    return out


def gemm_qkv_supported(x: torch.Tensor, w: torch.Tensor, cache: torch.Tensor, num_heads: int,
                       table: Optional[torch.Tensor]) -> bool:
    """True if gemm_qkv takes these operands: bfloat16, heads of 128, more than 64 rows, a rotation
    (if any) over the whole head."""
    lib = load_library()
    if x.dtype not in _DT or w.dtype not in _DT or cache.dim() != 5 or cache.dtype != torch.bfloat16:
        return False
    Hkv, P, D = cache.shape[2], cache.shape[3], cache.shape[4]
    if w.shape[0] != (int(num_heads) + 2 * Hkv) * D or (table is not None and table.shape[1] != D):
        return False
    return bool(lib.qe_gemm_qkv_supported(x.shape[0], x.shape[1], int(num_heads), Hkv, D, P, _DT[x.dtype], _DT[w.dtype]))


def gemm_qkv(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], num_heads: int, cache: torch.Tensor,
             positions: Optional[torch.Tensor], q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
             eps: float, table: Optional[torch.Tensor], slots: Optional[torch.Tensor],
             q_out: Optional[torch.Tensor] = None, tile: int = 0) -> torch.Tensor:
    """The q|k|v product x [T, K] . w [(Hq + 2 Hkv) D, K]^T (+ bias) with the step after it in its
    epilogue: per-head q/k RMSNorm (weights or None), half-split rotation from ``table`` (rows
    [cos | sin] per position, or None), q to the returned [T, Hq, D], k and v into ``cache``
    [pages, 2, Hkv, P, D] at ``slots`` (negative or no slots: nowhere).  The same results as gemm
    followed by qk_rope_store.  Needs gemm_qkv_supported."""
    lib = load_library()
    _need(x, "x", torch.bfloat16, (None, None))
    T, K = x.shape
    dev = x.device
    _need(cache, "cache", torch.bfloat16, (None, 2, None, None, None), dev)
    Hq, Hkv, P, D = int(num_heads), cache.shape[2], cache.shape[3], cache.shape[4]
    _need(w, "w", torch.bfloat16, ((Hq + 2 * Hkv) * D, K), dev)
    if not gemm_qkv_supported(x, w, cache, Hq, table):
        raise KernelError("gemm_qkv: operands not taken")
    if bias is not None:
        _need(bias, "bias", torch.float32, ((Hq + 2 * Hkv) * D,), dev)
    if positions is not None:
        _need(positions, "positions", torch.int32, (T,), dev)
    if table is not None:
        if positions is None:
            raise KernelError("gemm_qkv: a rotation needs positions")
        _need(table, "table", torch.float32, (None, D), dev)
    if (q_weight is None) != (k_weight is None):
        raise KernelError("gemm_qkv: q and k norm weights come together")
    if q_weight is not None:
        _need(q_weight, "q_weight", torch.float32, (D,), dev)
        _need(k_weight, "k_weight", torch.float32, (D,), dev)
    if slots is not None:
        _need(slots, "slots", torch.int32, (T,), dev)
    if q_out is None:
        q_out = torch.empty((T, Hq, D), dtype=torch.bfloat16, device=dev)
    _need(q_out, "q_out", torch.bfloat16, (T, Hq, D), dev)
    _check(lib.qe_gemm_qkv_run(x.data_ptr(), w.data_ptr(), _ptr(bias), T, K, Hq, Hkv, P, _ptr(positions), _ptr(slots),
                               _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(table), q_out.data_ptr(),
                               cache.data_ptr(), int(tile), _stream()), "gemm (q|k|v with norm, rotation, cache write)")
    return q_out


def qk_rope_store(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                  positions: Optional[torch.Tensor], q_weight: Optional[torch.Tensor],
                  k_weight: Optional[torch.Tensor], eps: float, table: Optional[torch.Tensor],
                  slots: Optional[torch.Tensor], cache: Optional[torch.Tensor], page_size: int,
                  q_out: Optional[torch.Tensor] = None, packed: bool = False) -> torch.Tensor:
    """Per-head q/k norm (if weights), rotation (if table), cache write (if slots) of qkv
    [T, (Hq + 2 Hkv) D].  cache: one layer's pages [pages, 2, Hkv, P, D].  Returns q [T, Hq, D];
    with ``packed`` it returns all heads [T, Hq + 2 Hkv, D] instead and writes no cache.
    The caller guarantees positions < table rows and slots < pages * P."""
    lib = load_library()
    T = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _need(qkv, "qkv", _ACT, (T, width))
    dev = qkv.device
    if positions is not None:
        _need(positions, "positions", torch.int32, (T,), dev)
    if (q_weight is None) != (k_weight is None):
        raise KernelError("qk_rope_store: q and k norm weights come together")
    if q_weight is not None:
        _need(q_weight, "q_weight", torch.float32, (head_dim,), dev)
        _need(k_weight, "k_weight", torch.float32, (head_dim,), dev)
    rotary_dim = 0
    if table is not None:
        _need(table, "table", torch.float32, (None, None), dev)
        rotary_dim = table.shape[1]
        if positions is None:
            raise KernelError("qk_rope_store: a rotation needs positions")
    if slots is not None:
        _need(slots, "slots", torch.int32, (T,), dev)
        if cache is None:
            raise KernelError("qk_rope_store: slots without a cache")
        _need(cache, "cache", qkv.dtype, (None, 2, num_kv_heads, page_size, head_dim), dev)
    packed_out = None
    if packed:
        if slots is not None:
            raise KernelError("qk_rope_store: the packed form writes no cache")
        packed_out = torch.empty((T, num_heads + 2 * num_kv_heads, head_dim), dtype=qkv.dtype, device=dev)
    else:
        if q_out is None:
            q_out = torch.empty((T, num_heads, head_dim), dtype=qkv.dtype, device=dev)
        _need(q_out, "q_out", qkv.dtype, (T, num_heads, head_dim), dev)
    _check(lib.qe_qk_rope_store(qkv.data_ptr(), _ptr(positions), _ptr(q_weight), _ptr(k_weight),
                                float(eps), _ptr(table), rotary_dim, _ptr(slots), _ptr(cache),
                                _ptr(q_out), _ptr(packed_out), T, num_heads, num_kv_heads, head_dim,
                                page_size, _DT[qkv.dtype], _stream()), "qk_rope_store")
    return packed_out if packed else q_out


def gemm_branch_splits(x: torch.Tensor, w: torch.Tensor) -> int:
    """How a product whose result goes to a norm that adds it to the stream should be asked for:
    0 = plain, S >= 1 = gemm(..., epilogue=EPI_PARTIAL, splits=S), the S partial products being
    what that norm takes as ``delta`` (few rows; many rows against a narrow matrix with a long K)."""
    lib = load_library()
    if x.dtype not in _DT or w.dtype not in _DT:
        return 0
    return int(lib.qe_gemm_branch_splits(x.shape[0], w.shape[0], x.shape[1], _DT[x.dtype], _DT[w.dtype]))


def gemm_branch_splits_for(rows: int, w: torch.Tensor, x_dtype: torch.dtype) -> int:
    """gemm_branch_splits for ``rows`` rows of x_dtype that are yet to be computed."""
    lib = load_library()
    if x_dtype not in _DT or w.dtype not in _DT:
        return 0
    return int(lib.qe_gemm_branch_splits(int(rows), w.shape[0], w.shape[1], _DT[x_dtype], _DT[w.dtype]))


def gemm_partial_preferred(x: torch.Tensor, w: torch.Tensor) -> bool:
    """True if the product of these operands is quickest cut along K into partial products
    (EPI_PARTIAL): more than 16 and at most 64 rows against a matrix of 16 M elements or more."""
    lib = load_library()
    return bool(lib.qe_gemm_partial_preferred(x.shape[0], w.shape[0], x.shape[1], _DT[x.dtype], _DT[w.dtype]))


def qk_rope_store_parts_supported(head_dim: int, table: Optional[torch.Tensor]) -> bool:
    """True if qk_rope_store_parts takes this head size and rotation table."""
    lib = load_library()
    return bool(lib.qe_qk_rope_store_parts_supported(int(head_dim), 0 if table is None else table.shape[1]))


def qk_rope_store_parts(parts: torch.Tensor, bias: Optional[torch.Tensor], num_heads: int, num_kv_heads: int,
                        head_dim: int, positions: Optional[torch.Tensor], q_weight: Optional[torch.Tensor],
                        k_weight: Optional[torch.Tensor], eps: float, table: Optional[torch.Tensor],
                        slots: Optional[torch.Tensor], cache: Optional[torch.Tensor], page_size: int) -> torch.Tensor:
    """qk_rope_store on a projection that comes as float32 partial products [S, T, (Hq + 2 Hkv) D]
    (gemm with EPI_PARTIAL): they are added in the order of S, with ``bias`` [width] if given, and
    rounded to bfloat16 before the norm, as the product would have stored them.  Returns q
    [T, Hq, D] bfloat16; cache: one layer's bfloat16 pages."""
    lib = load_library()
    width = (num_heads + 2 * num_kv_heads) * head_dim
    _need(parts, "parts", torch.float32, (None, None, width))
    S, T, dev = parts.shape[0], parts.shape[1], parts.device
    if not qk_rope_store_parts_supported(head_dim, table):
        raise KernelError("qk_rope_store_parts: head size or rotation not taken")
    if bias is not None:
        _need(bias, "bias", torch.float32, (width,), dev)
    if positions is not None:
        _need(positions, "positions", torch.int32, (T,), dev)
    if (q_weight is None) != (k_weight is None):
        raise KernelError("qk_rope_store_parts: q and k norm weights come together")
    if q_weight is not None:
        _need(q_weight, "q_weight", torch.float32, (head_dim,), dev)
        _need(k_weight, "k_weight", torch.float32, (head_dim,), dev)
    rotary_dim = 0
    if table is not None:
        _need(table, "table", torch.float32, (None, head_dim), dev)
        rotary_dim = head_dim
        if positions is None:
            raise KernelError("qk_rope_store_parts: a rotation needs positions")
    if slots is not None:
        _need(slots, "slots", torch.int32, (T,), dev)
        if cache is None:
            raise KernelError("qk_rope_store_parts: slots without a cache")
        _need(cache, "cache", torch.bfloat16, (None, 2, num_kv_heads, page_size, head_dim), dev)
    q_out = torch.empty((T, num_heads, head_dim), dtype=torch.bfloat16, device=dev)
    _check(lib.qe_qk_rope_store_parts(parts.data_ptr(), S, _ptr(bias), _ptr(positions), _ptr(q_weight), _ptr(k_weight),
                                      float(eps), _ptr(table), rotary_dim, _ptr(slots), _ptr(cache), q_out.data_ptr(),
                                      T, num_heads, num_kv_heads, head_dim, page_size, _stream()), "qk_rope_store_parts")
    return q_out


def use_matrix_f32(on: bool) -> None:
    """The float32 mode's attention and products on the matrix units (the default), or on the vector
    units' kernels, which sum in another order (for comparing the two)."""
    load_library().qe_use_matrix_f32(int(bool(on)))


def attention_decode_supported(q: torch.Tensor, cache: torch.Tensor) -> bool:
    """True if the MFMA decode kernel takes these sizes (bfloat16, head size 64 or 128, pages of a
    multiple of 16 tokens, at most 16 query heads per key/value head)."""
    lib = load_library()
    return bool(lib.qe_attention_decode_supported(q.shape[1], cache.shape[2], q.shape[2], cache.shape[3],
                                                  _DT[q.dtype]))


def attention_prefill_supported(q: torch.Tensor, cache: torch.Tensor) -> bool:
    """True if the MFMA prefill kernel takes these sizes: those of the decode kernel with a page
    size that is a power of two."""
    lib = load_library()
    return bool(lib.qe_attention_prefill_supported(q.shape[1], cache.shape[2], q.shape[2], cache.shape[3],
                                                   _DT[q.dtype]))


def prefill_tile_rows(num_heads: int, num_kv_heads: int) -> int:
    """Rows of a tile of the prefill attention kernel for these head counts (``other_tiles``)."""
    return load_library().qe_attention_prefill_rows(num_heads, num_kv_heads)


def prefill_tiles_on_device(portions: torch.Tensor, rows_per_tile: int, max_groups: int) -> torch.Tensor:
    """The ``other_tiles`` of attention() for portions int32 [n, 2] = (first row, rows) that lie on the
    device (a recorded step does not know them on the host): int32 [4 * max_groups, 2], groups of no rows
    beyond what the portions need.  The caller guarantees that the portions need at most max_groups
    groups of four tiles (every portion: ceil(rows / (4 * rows_per_tile)))."""
    lib = load_library()
    _need(portions, "portions", torch.int32, (None, 2))
    tiles = torch.empty((4 * int(max_groups), 2), dtype=torch.int32, device=portions.device)
    _check(lib.qe_attention_prefill_tiles_run(portions.data_ptr(), portions.shape[0], int(rows_per_tile),
                                              tiles.data_ptr(), int(max_groups), _stream()), "prefill tiles")
    return tiles


def prefill_uncut_keys() -> int:
    """Up to this many keys a row sees, the prefill attention kernel never cuts its walks into
    segments of keys."""
    return load_library().qe_attention_prefill_plan_uncut_keys()


def attention(q: torch.Tensor, cache: torch.Tensor, positions: torch.Tensor, tok_seq: torch.Tensor,
              block_table: torch.Tensor, scale: float, window: int = 0,
              out: Optional[torch.Tensor] = None, algo: int = ALGO_AUTO,
              dec_tokens: Optional[torch.Tensor] = None, max_dec_position: int = 0,
              other_tokens: Optional[torch.Tensor] = None,
              other_tiles: Optional[torch.Tensor] = None, prefill_groups: int = 0,
              max_other_keys: int = 0, prefill_segment_keys: int = -1,
              other_keys_row: Optional[int] = None, shared_keys: Optional[torch.Tensor] = None,
              keep_first: int = 0, sink: bool = False, chunk: int = 0) -> torch.Tensor:
    """q [T, Hq, D]; cache [pages, 2, Hkv, P, D] (key tiles [P][D], value tiles transposed [D][P]);
    positions, tok_seq int32 [T]; block_table int32 [B, max_blocks].  Token t sees the keys at
    positions max(0, p - window + 1) .. p of request tok_seq[t] (window 0: all).  The caller
    guarantees that those positions have pages in the table.  With ``keep_first`` the request's first
    keep_first keys are seen as well, wherever the window stands; with ``sink`` the softmax has a 1 added
    to its denominator (one more entry of score 0 that carries no value).  Both go with uncut walks of the
    prefill kernel only (no segments of keys).

    dec_tokens (int32 rows of q that are the single new token of their request, the largest of
    their positions being max_dec_position) go to the decode kernel where it takes the sizes;
    other_tokens are the remaining rows, and other_tiles (int32 [tiles, 2]: first row, number of
    rows <= prefill_tile_rows(Hq, Hkv), consecutive tokens of one request) the same rows cut
    for the prefill kernel (prefill_groups: its wave groups a block, 1 or 2, 0 to let it choose).
    max_other_keys: no row of other_tiles sees more keys than this (its position + 1); when given,
    the prefill kernel may cut long walks of few blocks into segments of keys (prefill_segment_keys:
    their length, a multiple of 64; 0 for none; -1 to let it choose).  A caller that does not know
    the positions (a recorded step) names the row of q that sees the most keys instead
    (other_keys_row): the kernel then cuts by that row's position.
    Without the lists every row is treated alike.

    ``chunk`` (instead of a window): positions are cut into chunks of that many, counted from the request's
    start, and a token sees the keys of its own chunk up to itself.

    shared_keys (int32, an entry per row of block_table, or None): how many of a request's first keys
    other requests read too.  A hint for the decode kernel's loads; results do not depend on it."""
    lib = load_library()
    _need(q, "q", _ACT, (None, None, None))
    T, Hq, D = q.shape
    dev = q.device
    _need(cache, "cache", q.dtype, (None, 2, None, None, D), dev)
    Hkv, P = cache.shape[2], cache.shape[3]
    _need(positions, "positions", torch.int32, (T,), dev)
    _need(tok_seq, "tok_seq", torch.int32, (T,), dev)
    _need(block_table, "block_table", torch.int32, (None, None), dev)
    if out is None:
        out = torch.empty_like(q)
    _need(out, "out", q.dtype, (T, Hq, D), dev)
    if Hq % Hkv:
        raise KernelError(f"attention: {Hq} query heads are no multiple of {Hkv} key/value heads")
    max_blocks = block_table.shape[1]
    if shared_keys is not None:
        _need(shared_keys, "shared_keys", torch.int32, (block_table.shape[0],), dev)
    if chunk:
        if window or keep_first or chunk < 0:
            raise KernelError("attention: chunks go without a window and kept first keys")
        window = -int(chunk)        # (the kernels take a negative window as the length of a chunk)
    keep_first, sink = int(keep_first) if window > 0 else 0, int(bool(sink))
    if keep_first < 0:
        raise KernelError("attention: negative keep_first")
    if keep_first or sink or chunk:
        prefill_segment_keys = 0    # (no segments of keys: such walks are short)

    def generic(tokens):
        n = T if tokens is None else tokens.shape[0]
        _check(lib.qe_attention(q.data_ptr(), out.data_ptr(), cache.data_ptr(), positions.data_ptr(),
                                tok_seq.data_ptr(), block_table.data_ptr(), max_blocks, _ptr(tokens), n,
                                Hq, Hkv, D, P, float(scale), int(window), keep_first, sink, _DT[q.dtype], _stream()),
               "attention")

    if dec_tokens is None and other_tokens is None:
        generic(None)
        return out
    if dec_tokens is not None and dec_tokens.shape[0]:
        _need(dec_tokens, "dec_tokens", torch.int32, (None,), dev)
        n_dec = dec_tokens.shape[0]
        if algo != ALGO_GENERIC and attention_decode_supported(q, cache):
            nbytes = lib.qe_attention_decode_workspace_bytes(n_dec, Hq, D, int(max_dec_position), DECODE_SPLIT_KEYS)
            ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
            _check(lib.qe_attention_decode_run(q.data_ptr(), out.data_ptr(), cache.data_ptr(),
                                               dec_tokens.data_ptr(), n_dec, positions.data_ptr(),
                                               tok_seq.data_ptr(), block_table.data_ptr(), max_blocks,
                                               _ptr(shared_keys), Hq, Hkv,
                                               D, P, float(scale), int(window), keep_first, sink, int(max_dec_position),
                                               DECODE_SPLIT_KEYS, ws.data_ptr(), nbytes, _stream()),
                   "attention (decode)")
        else:
            generic(dec_tokens)
    if other_tokens is not None and other_tokens.shape[0]:
        _need(other_tokens, "other_tokens", torch.int32, (None,), dev)
        if other_tiles is not None and algo != ALGO_GENERIC and attention_prefill_supported(q, cache):
            _need(other_tiles, "other_tiles", torch.int32, (None, 2), dev)
            n_tiles, max_keys, seg, ws, nbytes = other_tiles.shape[0], int(max_other_keys), 0, None, 0
            keys_row = -1
            if other_keys_row is not None:
                if not 0 <= int(other_keys_row) < T or max_keys > 0:
                    raise KernelError(f"attention: other_keys_row {other_keys_row} (of {T} rows) stands instead of max_other_keys")
                ks = lib.qe_attention_prefill_plan_segments(n_tiles, Hq, Hkv) if prefill_segment_keys else 1
                if ks > 1:
                    seg, keys_row = -ks, int(other_keys_row)
                    nbytes = lib.qe_attention_prefill_workspace_bytes_for(n_tiles, Hq, Hkv, D, ks)
                    ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
            elif max_keys > 0:
                seg = int(prefill_segment_keys)
                if seg < 0:
                    seg = lib.qe_attention_prefill_plan(n_tiles, Hq, Hkv, max_keys)
                if seg >= max_keys:
                    seg = 0
            elif prefill_segment_keys > 0:
                raise KernelError("attention: segments of keys need max_other_keys")
            if seg > 0:
                nbytes = lib.qe_attention_prefill_workspace_bytes(n_tiles, Hq, Hkv, D, max_keys, seg)
                ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
            _check(lib.qe_attention_prefill_run(q.data_ptr(), out.data_ptr(), cache.data_ptr(),
                                                other_tiles.data_ptr(), n_tiles,
                                                positions.data_ptr(), tok_seq.data_ptr(), block_table.data_ptr(),
                                                max_blocks, Hq, Hkv, D, P, float(scale), int(window), keep_first, sink,
                                                int(prefill_groups), seg, max_keys, keys_row, _ptr(ws), nbytes,
                                                _stream()),
                   "attention (prefill)")
        else:
            generic(other_tokens)
    return out


def attention_decode_fused_supported(qkv: torch.Tensor, cache: torch.Tensor, num_heads: int,
                                     table: Optional[torch.Tensor]) -> bool:
    """True if attention_decode_fused takes these operands: the sizes of the decode kernel, and a
    rotation (if any) over the whole head."""
    lib = load_library()
    D = cache.shape[4]
    return (qkv.dtype == torch.bfloat16 and (table is None or table.shape[1] == D) and
            bool(lib.qe_attention_decode_supported(num_heads, cache.shape[2], D, cache.shape[3], _DT[qkv.dtype])))


def attention_decode_fused(qkv: torch.Tensor, num_heads: int, cache: torch.Tensor, positions: torch.Tensor,
                           tok_seq: torch.Tensor, block_table: torch.Tensor, scale: float, window: int,
                           dec_tokens: Optional[torch.Tensor], max_dec_position: int,
                           q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                           table: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                           out: Optional[torch.Tensor] = None,
                           shared_keys: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of single new tokens with the step before it inside: per-head q/k RMSNorm
    (weights or None), half-split rotation from ``table`` (rows [cos | sin] of the head size, or
    None) and the write of each token's key and value to cache slot ``slots[t]`` (negative or no
    slots: not written).  qkv [T, (Hq + 2 Hkv) D] bfloat16; the rows ``dec_tokens`` (None: all
    rows) are computed into out [T, Hq, D]; the cache holds each request's keys before the
    token's own position.  shared_keys: as for attention()."""
    lib = load_library()
    _need(qkv, "qkv", torch.bfloat16, (None, None))
    T, dev = qkv.shape[0], qkv.device
    _need(cache, "cache", torch.bfloat16, (None, 2, None, None, None), dev)
    Hkv, P, D = cache.shape[2], cache.shape[3], cache.shape[4]
    Hq = int(num_heads)
    if qkv.shape[1] != (Hq + 2 * Hkv) * D:
        raise KernelError(f"attention_decode_fused: qkv rows of {qkv.shape[1]} are not ({Hq} + 2 * {Hkv}) * {D}")
    if not attention_decode_fused_supported(qkv, cache, Hq, table):
        raise KernelError("attention_decode_fused: sizes not taken")
    _need(positions, "positions", torch.int32, (T,), dev)
    _need(tok_seq, "tok_seq", torch.int32, (T,), dev)
    _need(block_table, "block_table", torch.int32, (None, None), dev)
    if dec_tokens is not None:
        _need(dec_tokens, "dec_tokens", torch.int32, (None,), dev)
    if q_weight is not None:
        _need(q_weight, "q_weight", torch.float32, (D,), dev)
    if k_weight is not None:
        _need(k_weight, "k_weight", torch.float32, (D,), dev)
    if table is not None:
        _need(table, "table", torch.float32, (None, D), dev)
    if slots is not None:
        _need(slots, "slots", torch.int32, (T,), dev)
    if shared_keys is not None:
        _need(shared_keys, "shared_keys", torch.int32, (block_table.shape[0],), dev)
    if out is None:
        out = torch.empty((T, Hq, D), dtype=torch.bfloat16, device=dev)
    _need(out, "out", torch.bfloat16, (T, Hq, D), dev)
    n_dec = dec_tokens.shape[0] if dec_tokens is not None else T
    if n_dec == 0:
        return out
    nbytes = lib.qe_attention_decode_workspace_bytes(n_dec, Hq, D, int(max_dec_position), DECODE_SPLIT_KEYS)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
    _check(lib.qe_attention_decode_fused_run(qkv.data_ptr(), out.data_ptr(), cache.data_ptr(), _ptr(dec_tokens),
                                             n_dec, positions.data_ptr(), tok_seq.data_ptr(), block_table.data_ptr(),
                                             block_table.shape[1], _ptr(shared_keys), _ptr(slots), _ptr(q_weight),
                                             _ptr(k_weight),
                                             float(eps), _ptr(table), Hq, Hkv, D, P, float(scale), int(window),
                                             int(max_dec_position), DECODE_SPLIT_KEYS, ws.data_ptr(), nbytes,
                                             _stream()), "attention (decode, fused)")
    return out


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Lowest index of the largest logit per row; logits float32 [R, V] -> int32 [R]."""
    lib = load_library()
    _need(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _need(out, "out", torch.int32, (R,), logits.device)
    nbytes = lib.qe_argmax_workspace_bytes(R, V)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=logits.device) if nbytes else None
    _check(lib.qe_argmax(logits.data_ptr(), out.data_ptr(), R, V, _ptr(ws), nbytes, _stream()), "argmax")
    return out


def argmax_static_takes(rows: int, vocab: int) -> bool:
    """True if argmax_static takes logits of this shape (what lies between its two stages fits the
    library's fixed buffer)."""
    lib = load_library()
    return lib.qe_argmax_workspace_bytes(int(rows), int(vocab)) <= lib.qe_argmax_static_max_bytes()


def argmax_static(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """argmax into ``out`` (int32 [R]) without any allocation: what lies between the two stages is kept
    in a buffer inside the library (one per GPU, shared by all calls on it: calls on one stream only).
    For code that is recorded into a graph; needs argmax_static_takes(R, V)."""
    lib = load_library()
    _need(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    _need(out, "out", torch.int32, (R,), logits.device)
    _check(lib.qe_argmax_static(logits.data_ptr(), out.data_ptr(), R, V, _stream()), "argmax (static)")
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Inverse-CDF draw from softmax(logits / temperature) per row with uniform[r] in [0, 1).
    Every temperature must be positive."""
    lib = load_library()
    _need(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    _need(temperature, "temperature", torch.float32, (R,), logits.device)
    _need(uniform, "uniform", torch.float32, (R,), logits.device)
    if out is None:
        out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _need(out, "out", torch.int32, (R,), logits.device)
    _check(lib.qe_sample(logits.data_ptr(), temperature.data_ptr(), uniform.data_ptr(), out.data_ptr(),
                         R, V, _stream()), "sample")
    return out


def mfma_probe(blocks: int = 512, iters: int = 20000, device="cuda:0") -> float:
    """Floating-point operations a second that register-resident bfloat16 MFMAs (32 x 32 x 16) reach
    on this device, eight waves a compute unit with 512 blocks: a measured peak, for scale."""
    lib = load_library()
    out = torch.empty(blocks * 256, dtype=torch.float32, device=device)
    flops = ctypes.c_double(0.0)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = 0.0
    for rep in range(3):                                   # (the first repetition brings the clock up)
        start.record()
        _check(lib.qe_mfma_probe(out.data_ptr(), int(blocks), int(iters), ctypes.byref(flops), _stream()), "mfma probe")
        end.record()
        end.synchronize()
        best = max(best, flops.value / (start.elapsed_time(end) * 1e-3))
    return best


# ---- norm after the residual sum, the short convolution, the polynomial activation ------------------
def postnorm(x: torch.Tensor, delta: Optional[torch.Tensor], alpha: float, gain: torch.Tensor, eps: float,
             act_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """x <- gain * z / sqrt(mean(z^2) + eps) with z = alpha * x + delta, on the 32-bit stream x [T, H], in
    place.  delta: None, [T, H] (bfloat16 or float32) or float32 [S, T, H], added in the order of S.  gain:
    float32 [1] (one for all coordinates) or [H].  With ``act_dtype`` bfloat16 a copy of the new x in that type is returned (what the next
    products read); with float32 or None, nothing (the stream itself is read)."""
    lib = load_library()
    _need(x, "x", torch.float32, (None, None))
    T, H = x.shape
    _need(gain, "gain", torch.float32, (None,), x.device)
    if gain.shape[0] not in (1, H):
        raise KernelError(f"postnorm: {gain.shape[0]} gains for rows of {H}")
    n_delta, dt_d = 0, F32
    if delta is not None:
        if delta.dim() == 3:
            _need(delta, "delta", torch.float32, (None, T, H), x.device)
            n_delta = delta.shape[0]
        else:
            _need(delta, "delta", _ACT, (T, H), x.device)
            n_delta, dt_d = 1, _DT[delta.dtype]
    act = None
    if act_dtype == torch.bfloat16:
        act = torch.empty((T, H), dtype=torch.bfloat16, device=x.device)
    _check(lib.qe_postnorm(x.data_ptr(), _ptr(delta), n_delta, dt_d, float(alpha), gain.data_ptr(), gain.shape[0], float(eps),
                           _ptr(act), BF16 if act is not None else F32, T, H, _stream()), "postnorm")
    return act


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e per row of z (float32 [T, F]), rms(v) =
    sqrt(mean(v^2) + eps), coef = (a, b, c, e) float32 [4]; all in 32-bit, one rounding at the store."""
    lib = load_library()
    _need(z, "z", torch.float32, (None, None))
    T, Fd = z.shape
    _need(coef, "coef", torch.float32, (4,), z.device)
    out = torch.empty((T, Fd), dtype=out_dtype, device=z.device)
    _check(lib.qe_polynorm(z.data_ptr(), coef.data_ptr(), float(eps), out.data_ptr(), _DT[out_dtype], T, Fd, _stream()),
           "polynorm")
    return out


def short_conv(x: torch.Tensor, w: torch.Tensor, state: Optional[torch.Tensor], tok_seq: torch.Tensor,
               out_dtype: torch.dtype, update: bool = True, single_rows: bool = False) -> torch.Tensor:
    """out_t = x_t + sum_k w[:, taps - 1 - k] x_(t - k) along each request's tokens, x the 32-bit stream
    [T, H], w float32 [H, taps].  What lies before a request's rows in this step comes from state
    (float32 [slots, taps - 1, H], row tok_seq[t]: the request's last taps - 1 inputs), which then takes
    the step's last inputs (``update``).  The rows of a request are consecutive.  ``single_rows``: the caller
    knows that no two rows belong to the same request (single new tokens, each with a state row of its own):
    convolution and update are then one launch."""
    lib = load_library()
    _need(x, "x", torch.float32, (None, None))
    T, H = x.shape
    _need(w, "w", torch.float32, (H, None), x.device)
    taps = w.shape[1]
    _need(tok_seq, "tok_seq", torch.int32, (T,), x.device)
    if taps > 1:
        if state is None:
            raise KernelError("short_conv: no state")
        _need(state, "state", torch.float32, (None, taps - 1, H), x.device)
    out = torch.empty((T, H), dtype=out_dtype, device=x.device)
    _check(lib.qe_short_conv(x.data_ptr(), w.data_ptr(), _ptr(state), tok_seq.data_ptr(), out.data_ptr(),
                             _DT[out_dtype], T, H, taps, 2 if (update and single_rows) else int(update), _stream()),
           "short_conv")
    return out


# ---- attention over one cached latent per token --------------------------------------------------------
def latent_kv_store(kv: torch.Tensor, weight: torch.Tensor, eps: float, positions: torch.Tensor,
                    inv_freq: torch.Tensor, slots: Optional[torch.Tensor], cache: torch.Tensor,
                    q: Optional[torch.Tensor] = None, qp: Optional[torch.Tensor] = None, dim: int = 0,
                    half_split: bool = False) -> None:
    """kv float32 [T, R + Dr] (R = weight's length): the first R normed (weight * u / rms(u)), the last Dr
    turned in neighbouring pairs (``half_split``: number i with number i + n) by positions * inv_freq (float32 [n],
    2 n <= Dr; the rest passes), into
    the row slots[t] of cache [pages, 1, 1, P, R + Dr] (negative slot, or no slots: nowhere).  With q
    [T, H, dim + Dr] and qp [T, H, R + Dr] the same launch does what latent_q_rotate does."""
    lib = load_library()
    _need(kv, "kv", torch.float32, (None, None))
    T, D = kv.shape
    dev = kv.device
    _need(weight, "weight", torch.float32, (None,), dev)
    R = weight.shape[0]
    _need(cache, "cache", _ACT, (None, 1, 1, None, D), dev)
    _need(positions, "positions", torch.int32, (T,), dev)
    if slots is not None:
        _need(slots, "slots", torch.int32, (T,), dev)
    _need(inv_freq, "inv_freq", torch.float32, (None,), dev)
    H = 0
    if q is not None:
        _need(q, "q", cache.dtype, (T, None, int(dim) + D - R), dev)
        H = q.shape[1]
        _need(qp, "qp", cache.dtype, (T, H, D), dev)
    _check(lib.qe_latent_kv_store(kv.data_ptr(), weight.data_ptr(), float(eps), positions.data_ptr(),
                                  inv_freq.data_ptr(), 2 * inv_freq.shape[0], _ptr(slots), cache.data_ptr(),
                                  _DT[cache.dtype], T, R, D - R, _ptr(q), _ptr(qp), H, int(dim), int(bool(half_split)),
                                  _stream()), "latent_kv_store")


def latent_q_rotate(q: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, qp: torch.Tensor,
                    dim: int, half_split: bool = False) -> None:
    """q [T, H, dim + Dr] -> the last Dr of each head, turned as in latent_kv_store, into the last Dr of
    qp [T, H, R + Dr]."""
    lib = load_library()
    _need(q, "q", _ACT, (None, None, None))
    T, H, Dq = q.shape
    Dr = Dq - int(dim)
    _need(qp, "qp", q.dtype, (T, H, None), q.device)
    R = qp.shape[2] - Dr
    if Dr < 0 or R <= 0:
        raise KernelError("latent_q_rotate: sizes do not fit")
    if Dr == 0:
        return
    _need(positions, "positions", torch.int32, (T,), q.device)
    _need(inv_freq, "inv_freq", torch.float32, (None,), q.device)
    _check(lib.qe_latent_q_rotate(q.data_ptr(), positions.data_ptr(), inv_freq.data_ptr(), 2 * inv_freq.shape[0],
                                  qp.data_ptr(), _DT[q.dtype], T, H, int(dim), Dr, R, int(bool(half_split)), _stream()),
           "latent_q_rotate")


def latent_attention(qp: torch.Tensor, cache: torch.Tensor, positions: torch.Tensor, tok_seq: torch.Tensor,
                     block_table: torch.Tensor, latent: int, scale: float, algo: int = ALGO_AUTO,
                     window: int = 0, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """qp [T, H, R + Dr], cache [pages, 1, 1, P, R + Dr]: per (token, head) softmax(scale * qp . rows) . rows[:R]
    over the rows at positions 0 .. p of request tok_seq[t] (``window`` > 0: at p - window + 1 .. p) -> [T, H, R].
    ``sink`` (float32 [H]): exp(sink[h]) joins the softmax's denominator, one more entry that carries no value.  32-bit scores and weights.  The rows
    of a request are consecutive and their positions rise.  bfloat16 goes to the kernel on the matrix units
    where it takes the sizes (multiples of 8, a latent of at most 512; the weights are rounded to bfloat16
    before they meet the values), everything else (and ALGO_GENERIC) to the kernel on the vector units."""
    lib = load_library()
    _need(qp, "qp", _ACT, (None, None, None))
    T, H, D = qp.shape
    dev = qp.device
    R = int(latent)
    _need(cache, "cache", qp.dtype, (None, 1, 1, None, D), dev)
    P = cache.shape[3]
    _need(positions, "positions", torch.int32, (T,), dev)
    _need(tok_seq, "tok_seq", torch.int32, (T,), dev)
    _need(block_table, "block_table", torch.int32, (None, None), dev)
    window = int(window or 0)
    if window < 0:
        raise KernelError("latent_attention: a negative window")
    if sink is not None:
        _need(sink, "sink", torch.float32, (H,), dev)
    out = torch.empty((T, H, R), dtype=qp.dtype, device=dev)
    if qp.dtype == torch.bfloat16 and algo != ALGO_GENERIC and lib.qe_latent_attention_mfma_supported(R, D - R):
        nbytes = lib.qe_latent_attention_mfma_workspace_bytes(T, H, R, window)
        ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev) if nbytes else None
        _check(lib.qe_latent_attention_mfma(qp.data_ptr(), out.data_ptr(), cache.data_ptr(), positions.data_ptr(),
                                            tok_seq.data_ptr(), block_table.data_ptr(), block_table.shape[1], T, H, R,
                                            D - R, P, float(scale), window, _ptr(sink), _ptr(ws), nbytes, _stream()),
               "latent_attention (mfma)")
        return out
    _check(lib.qe_latent_attention(qp.data_ptr(), out.data_ptr(), cache.data_ptr(), positions.data_ptr(),
                                   tok_seq.data_ptr(), block_table.data_ptr(), block_table.shape[1], T, H, R, D - R, P,
                                   float(scale), window, _ptr(sink), _DT[qp.dtype], _stream()), "latent_attention")
    return out


def gemm_heads(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor] = None,
               algo: int = ALGO_AUTO) -> torch.Tensor:
    """out[t, h, :N] = w[h] x[t, h, :K] for w [H, N, K]; x [T, H, >= K] and out [T, H, >= N] (the product reads
    the first K and writes the first N numbers of each head).  gate [T, H * N]: the result times
    sigmoid(gate); gate [T, H] (or a view of H columns of wider rows): one gate per head."""
    lib = load_library()
    _need(w, "w", _ACT, (None, None, None))
    H, N, K = w.shape
    _need(x, "x", _ACT, (None, H, None))
    T = x.shape[0]
    _need(out, "out", x.dtype, (T, H, None), x.device)
    if x.shape[2] < K or out.shape[2] < N:
        raise KernelError("gemm_heads: heads narrower than the product")
    if x.dtype == torch.float32 and w.dtype != torch.float32:
        raise KernelError("gemm_heads: 32-bit activations need 32-bit weights")
    gs = (0, 0, 0)
    if gate is not None:
        if gate.dim() == 2 and gate.shape == (T, H) and gate.stride(1) == 1 and H * N != H:
            if not gate.is_cuda or gate.dtype != x.dtype or gate.device != x.device:
                raise KernelError("gemm_heads: the gate is not where and what the rows are")
            gs = (gate.stride(0), 1, 0)
        else:
            _need(gate, "gate", x.dtype, (T, H * N), x.device)
            gs = (H * N, N, 1)
    if (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and algo != ALGO_GENERIC and
            lib.qe_gemm_heads_mfma_supported(K, H * x.shape[2], x.shape[2])):
        _check(lib.qe_gemm_heads_mfma(x.data_ptr(), H * x.shape[2], x.shape[2], w.data_ptr(), out.data_ptr(),
                                      H * out.shape[2], out.shape[2], _ptr(gate), gs[0], gs[1], gs[2], T, H, N, K, _stream()),
               "gemm_heads (mfma)")
        return out
    _check(lib.qe_gemm_heads(x.data_ptr(), H * x.shape[2], x.shape[2], w.data_ptr(), out.data_ptr(),
                             H * out.shape[2], out.shape[2], _ptr(gate), gs[0], gs[1], gs[2], T, H, N, K, _DT[x.dtype], _DT[w.dtype],
                             _stream()), "gemm_heads")
    return out


# ---- mixture of experts -----------------------------------------------------------------------------------
def moe_route(logits: torch.Tensor, groups: int, keep: int, top: int):
    """logits float32 [T, E] -> (ids int32 [T, top], weights float32 [T, top]): softmax over all experts,
    the ``keep`` best of ``groups`` equal groups of neighbours (a group's score is its largest), the ``top``
    largest scores among them, as they are."""
    lib = load_library()
    _need(logits, "logits", torch.float32, (None, None))
    T, E = logits.shape
    ids = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    _check(lib.qe_moe_route(logits.data_ptr(), ids.data_ptr(), weights.data_ptr(), T, E, int(groups), int(keep),
                            int(top), _stream()), "moe_route")
    return ids, weights


def moe_route_biased(logits: torch.Tensor, correction: Optional[torch.Tensor], top: int, scale: float,
                     transposed: bool = False, logit_bias: Optional[torch.Tensor] = None, experts: int = 0):
    """logits float32 [T, E] (``transposed``: [E, T]), correction float32 [E] -> (ids int32 [T, top], weights float32 [T, top]): softmax
    over all experts; the ``top`` largest of score + correction are chosen (the lower index on ties); their
    weights are their scores without the correction, divided by the chosen scores' sum (+ 1e-20), times scale.
    Without a correction (None) the ``top`` largest logits are chosen and weighed by the softmax over them alone.
    ``logit_bias`` (float32 [E]) is added to the logits first.  ``experts``: only the first so many outputs of the
    logits are the router's (the rest belongs to the caller); 0: all."""
    lib = load_library()
    _need(logits, "logits", torch.float32, (None, None))
    T, ld = (logits.shape[1], 0) if transposed else logits.shape
    E = int(experts) or (logits.shape[0] if transposed else logits.shape[1])
    if E > (logits.shape[0] if transposed else logits.shape[1]):
        raise KernelError("moe_route_biased: more experts than logits")
    if correction is not None:
        _need(correction, "correction", torch.float32, (E,), logits.device)
    if logit_bias is not None:
        _need(logit_bias, "logit_bias", torch.float32, (E,), logits.device)
    ids = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    _check(lib.qe_moe_route_biased(logits.data_ptr(), _ptr(correction), ids.data_ptr(), weights.data_ptr(), T, E,
                                   int(top), float(scale), int(bool(transposed)), _ptr(logit_bias), int(ld), _stream()),
           "moe_route_biased")
    return ids, weights


def scale_(x: torch.Tensor, s: float) -> None:
    """x *= s on a 32-bit tensor."""
    lib = load_library()
    _need(x, "x", torch.float32)
    _check(lib.qe_scale_f32(x.data_ptr(), x.numel(), float(s), _stream()), "scale")


def qkv_conv_rope_store(qkv: torch.Tensor, conv_w: torch.Tensor, state: Optional[torch.Tensor], tok_seq: torch.Tensor,
                        positions: torch.Tensor, inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                        cache: torch.Tensor, num_heads: int, num_kv_heads: int, k_dim: int, v_dim: int,
                        single_rows: bool = False, conv_w_t: Optional[torch.Tensor] = None) -> torch.Tensor:
    """What stands between a q|k|v projection and the attention where q, k and v each pass a short causal
    convolution over time and q and k are then rotated on their first numbers.  qkv [T, Hq Dk + Hkv Dk + Hkv Dv];
    conv_w float32 [that many, taps]; state float32 [slots, taps - 1, that many] (row tok_seq[t]: the request's last
    projected rows; None for one tap), brought up to date; inv_freq float32 [rotated numbers / 2] or None.
    cache [pages, 2, Hkv, P, Dc] with Dc >= Dk, Dv: keys and values go to slots[t] (negative or no slots:
    nowhere), zeros beyond a head's own numbers.  Returns q [T, Hq, Dc], padded likewise.  The rows of a request
    are consecutive; ``single_rows``: no two rows belong to the same request (one launch).  ``conv_w_t``: conv_w
    transposed, float32 [taps, that many], for the kernel of many rows (eight channels a thread)."""
    lib = load_library()
    _need(qkv, "qkv", _ACT, (None, None))
    T, C = qkv.shape
    dev = qkv.device
    Hq, Hkv, Dk, Dv = int(num_heads), int(num_kv_heads), int(k_dim), int(v_dim)
    if C != Hq * Dk + Hkv * (Dk + Dv):
        raise KernelError(f"qkv_conv_rope_store: rows of {C} are not {Hq} x {Dk} + {Hkv} x ({Dk} + {Dv})")
    _need(conv_w, "conv_w", torch.float32, (C, None), dev)
    taps = conv_w.shape[1]
    if taps > 1:
        if state is None:
            raise KernelError("qkv_conv_rope_store: no state")
        _need(state, "state", torch.float32, (None, taps - 1, C), dev)
    _need(tok_seq, "tok_seq", torch.int32, (T,), dev)
    _need(positions, "positions", torch.int32, (T,), dev)
    rot = 0
    if inv_freq is not None:
        _need(inv_freq, "inv_freq", torch.float32, (None,), dev)
        rot = 2 * inv_freq.shape[0]
    _need(cache, "cache", qkv.dtype, (None, 2, Hkv, None, None), dev)
    P, Dc = cache.shape[3], cache.shape[4]
    if slots is not None:
        _need(slots, "slots", torch.int32, (T,), dev)
    if conv_w_t is not None:
        _need(conv_w_t, "conv_w_t", torch.float32, (taps, C), dev)
    q = torch.empty((T, Hq, Dc), dtype=qkv.dtype, device=dev)
    _check(lib.qe_qkv_conv_rope_store(qkv.data_ptr(), conv_w.data_ptr(), _ptr(conv_w_t), _ptr(state), tok_seq.data_ptr(),
                                      positions.data_ptr(), _ptr(inv_freq), _ptr(slots), q.data_ptr(), cache.data_ptr(),
                                      T, Hq, Hkv, Dk, Dv, Dc, P, taps, rot, int(bool(single_rows)), _DT[qkv.dtype],
                                      _stream()), "qkv_conv_rope_store")
    return q


def moe_experts(x: torch.Tensor, ids: Optional[torch.Tensor], weights: Optional[torch.Tensor], w_gate_up: torch.Tensor,
                w_down: torch.Tensor, limit: float = 0.0, slope: float = 1.0, interleaved: bool = False,
                algo: int = ALGO_AUTO, act: str = "gated", identity: int = 0,
                rows_dtype: torch.dtype = torch.float32, biased_route=None,
                parts_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The chosen experts' outputs, weighted: float32 [S, T, H] whose sum over S, in order, is the mixture's
    output (S = top: a token's choices in their order; or S = 1: already added up in that order).
    x [T, K]; w_gate_up [E, 2 F, K] (gate rows, then up rows; or, ``interleaved``, in alternating blocks of
    32 as interleave_gate_up lays them); w_down [E, H, F].  An expert: g = min(gate x, limit),
    u = clamp(up x, -limit, limit), down (g sigmoid(slope g) (u + 1)).  With ``act`` "relu_sq" the first
    matrix is one [E, F, K] and an expert is down (relu(up x)^2).  ``identity``: so many more
    experts, the ids E .. E + identity - 1, are the identity: their output is the token's row itself, times the weight.
    ``rows_dtype``: the element type in which the path of many pairs leaves an expert's output rows before they are
    weighed and added in 32-bit (float32, or bfloat16 with bfloat16 operands: half the bytes of the largest tensor of
    the mixture).  ``biased_route``: instead of ids and weights (both None), (logits float32 [T, E + identity],
    correction float32 [E + identity], top, scale[, transposed: the logits are [E + identity, T]]) for the routing of
    moe_route_biased (a None correction: the largest logits, weighed by the softmax over them alone; two more entries:
    a bias float32 [E + identity] that is added to the logits, and how many of the logits' outputs are the router's
    where they are the first of more): a step of few tokens then
    routes, sorts and writes the identity experts' rows in one launch.  ``limit`` 0: the plain silu(g) u.  ``parts_out``: float32 [top, T, H] to take the
    parts (the paths of fewer than 1024 pairs only).

    The (token, choice) pairs are grouped by expert on the device.  bfloat16 with many pairs: their rows are
    gathered side by side and both products run on the tiled kernel of the dense products, a tile of 128
    rows per block, every block finding its expert in the list of tiles.  bfloat16 with few pairs: a kernel
    that reads its rows in place, tiles of 16 or 64 rows.  Otherwise (and ALGO_GENERIC) the kernel on the
    vector units."""
    lib = load_library()
    _need(x, "x", _ACT, (None, None))
    T, K = x.shape
    dev = x.device
    if biased_route is not None:
        if ids is not None or weights is not None:
            raise KernelError("moe_experts: ids and weights, or a route to compute them, not both")
        r_logits, r_corr, top, r_scale = biased_route[:4]
        r_transposed = len(biased_route) > 4 and bool(biased_route[4])       # logits [E + identity, T]
        r_bias = biased_route[5] if len(biased_route) > 5 else None          # added to the logits (float32, an entry per output)
        top = int(top)
        _need(r_logits, "logits", torch.float32, (None, T) if r_transposed else (T, None), dev)
        r_width = r_logits.shape[0] if r_transposed else r_logits.shape[1]
        # (the router's outputs may be the first of more outputs of one product)
        r_outputs = int(biased_route[6]) if len(biased_route) > 6 and biased_route[6] else r_width
        if r_outputs > r_width:
            raise KernelError("moe_experts: more router outputs than logits")
        if r_corr is not None:
            _need(r_corr, "correction", torch.float32, (r_outputs,), dev)
        if r_bias is not None:
            _need(r_bias, "logit_bias", torch.float32, (r_outputs,), dev)
    else:
        _need(ids, "ids", torch.int32, (T, None), dev)
        top = ids.shape[1]
        _need(weights, "weights", torch.float32, (T, top), dev)
    _need(w_gate_up, "w_gate_up", x.dtype, (None, None, K), dev)
    E, F2 = w_gate_up.shape[0], w_gate_up.shape[1]
    if act not in ("gated", "relu_sq"):
        raise KernelError(f"moe_experts: activation {act!r}")
    single = act == "relu_sq"
    first_mode = 2 if single else 1
    Fd = F2 if single else F2 // 2
    _need(w_down, "w_down", x.dtype, (E, None, Fd), dev)
    Hout = w_down.shape[1]
    if interleaved and (Fd % 32 or single):
        raise KernelError("moe_experts: interleaved gate|up rows come in blocks of 32")
    identity = int(identity)
    if identity < 0 or (identity and Hout != K):
        raise KernelError("moe_experts: identity experts keep the width")
    n = T * top
    mfma = (x.dtype == torch.bfloat16 and algo != ALGO_GENERIC and lib.qe_moe_gemm_mfma_supported(K)
            and lib.qe_moe_gemm_mfma_supported(Fd))
    tiled = mfma and (interleaved or single) and n >= 1024 and K >= 64 and Fd >= 64
    if tiled:
        tile_rows = lib.qe_gemm_mfma_grouped_tile_rows()
    elif mfma:
        tile_rows = 16 if n <= 512 else 64
    else:
        tile_rows = lib.qe_moe_tile_rows()
    max_tiles = (n + tile_rows - 1) // tile_rows + min(E, n)
    meta = torch.empty(2 * n + 3 * max_tiles + 1, dtype=torch.int32, device=dev)
    perm, inv, tiles, n_tiles = meta[:n], meta[n:2 * n], meta[2 * n:2 * n + 3 * max_tiles], meta[2 * n + 3 * max_tiles:]
    fused_front = False
    parts = None
    if parts_out is not None:
        if tiled:
            raise KernelError("moe_experts: parts_out goes with fewer than 1024 pairs")
        _need(parts_out, "parts_out", torch.float32, (top, T, Hout), dev)
        parts = parts_out
    if biased_route is not None:
        if r_outputs != E + identity:
            raise KernelError(f"moe_experts: {r_outputs} router outputs for {E} experts and {identity} identity experts")
        if not tiled and not r_transposed and lib.qe_moe_front_small_supported(T, E + identity, top):
            # few tokens: routing, sort and the identity experts' rows in one launch
            ids = torch.empty((T, top), dtype=torch.int32, device=dev)
            weights = torch.empty((T, top), dtype=torch.float32, device=dev)
            if parts is None:
                parts = torch.empty((top, T, Hout), dtype=torch.float32, device=dev)
            _check(lib.qe_moe_front_small(r_logits.data_ptr(), _ptr(r_corr), x.data_ptr(), ids.data_ptr(),
                                          weights.data_ptr(), perm.data_ptr(), inv.data_ptr(), tiles.data_ptr(),
                                          n_tiles.data_ptr(), parts.data_ptr(), max_tiles, T, Hout, E + identity, E, top,
                                          float(r_scale), tile_rows, _DT[x.dtype], _ptr(r_bias), r_width, _stream()),
                   "moe_front_small")
            fused_front = True
        else:
            ids, weights = moe_route_biased(r_logits, r_corr, top, r_scale, transposed=r_transposed, logit_bias=r_bias,
                                            experts=r_outputs)
    # (identity experts are buckets of the sort like the others, behind them, and get no tiles)
    if not fused_front:
        _check(lib.qe_moe_sort(ids.data_ptr(), n, E + identity, E, tile_rows, perm.data_ptr(), inv.data_ptr(), tiles.data_ptr(),
                               n_tiles.data_ptr(), max_tiles, _stream()), "moe_sort")

    def identity(parts_, rows_):
        if identity and not fused_front:
            _check(lib.qe_moe_identity(x.data_ptr(), ids.data_ptr(), weights.data_ptr(), inv.data_ptr(), _ptr(parts_),
                                       _ptr(rows_), T, top, Hout, E, _DT[x.dtype],
                                       int(rows_ is not None and rows_.dtype == x.dtype and x.dtype != torch.float32),
                                       _stream()), "moe_identity")
    a = torch.empty((n, Fd), dtype=x.dtype, device=dev)
    if tiled:
        xs = torch.empty((n, K), dtype=x.dtype, device=dev)
        _check(lib.qe_moe_gather(x.data_ptr(), perm.data_ptr(), top, xs.data_ptr(), n, K, _DT[x.dtype], _stream()), "moe_gather")
        _check(lib.qe_gemm_mfma_grouped(xs.data_ptr(), w_gate_up.data_ptr(), a.data_ptr(), tiles.data_ptr(),
                                        n_tiles.data_ptr(), max_tiles, Fd if single else 2 * Fd, K, first_mode, float(limit),
                                        float(slope), BF16, _stream()), "grouped gemm (gate, up)")
        if rows_dtype not in (torch.float32, torch.bfloat16):
            raise KernelError(f"moe_experts: rows in {rows_dtype}")
        y = torch.empty((n, Hout), dtype=rows_dtype, device=dev)
        _check(lib.qe_gemm_mfma_grouped(a.data_ptr(), w_down.data_ptr(), y.data_ptr(), tiles.data_ptr(),
                                        n_tiles.data_ptr(), max_tiles, Hout, Fd, 0, 0.0, 1.0, _DT[rows_dtype], _stream()),
               "grouped gemm (down)")
        identity(None, y)
        out = torch.empty((1, T, Hout), dtype=torch.float32, device=dev)
        _check(lib.qe_moe_combine(y.data_ptr(), inv.data_ptr(), weights.data_ptr(), out.data_ptr(), T, top, Hout,
                                  _DT[rows_dtype], _stream()), "moe_combine")
        return out
    if parts is None:
        parts = torch.empty((top, T, Hout), dtype=torch.float32, device=dev)
    if mfma:
        _check(lib.qe_moe_gemm_mfma(x.data_ptr(), perm.data_ptr(), top, w_gate_up.data_ptr(), a.data_ptr(), None,
                                    tiles.data_ptr(), n_tiles.data_ptr(), max_tiles, tile_rows, T, Fd, K, float(limit),
                                    float(slope), first_mode, int(interleaved), _stream()), "moe_gemm (gate, up; mfma)")
        _check(lib.qe_moe_gemm_mfma(a.data_ptr(), perm.data_ptr(), top, w_down.data_ptr(), parts.data_ptr(),
                                    weights.data_ptr(), tiles.data_ptr(), n_tiles.data_ptr(), max_tiles, tile_rows, T,
                                    Hout, Fd, 0.0, 0.0, 0, 0, _stream()), "moe_gemm (down; mfma)")
        identity(parts, None)
        return parts
    _check(lib.qe_moe_gemm(x.data_ptr(), perm.data_ptr(), top, w_gate_up.data_ptr(), a.data_ptr(), None,
                           tiles.data_ptr(), n_tiles.data_ptr(), max_tiles, T, Fd, K, float(limit), float(slope), first_mode,
                           int(interleaved), _DT[x.dtype], _DT[w_gate_up.dtype], _stream()), "moe_gemm (gate, up)")
    _check(lib.qe_moe_gemm(a.data_ptr(), perm.data_ptr(), top, w_down.data_ptr(), parts.data_ptr(), weights.data_ptr(),
                           tiles.data_ptr(), n_tiles.data_ptr(), max_tiles, T, Hout, Fd, 0.0, 0.0, 0, 0,
                           _DT[x.dtype], _DT[w_down.dtype], _stream()), "moe_gemm (down)")
    identity(parts, None)
    return parts


# ---- queries, keys and values normed over the whole projection or per head; values from keys; blended values --------
QK_NORM_NONE, QK_NORM_HEAD, QK_NORM_WHOLE = 0, 1, 2


def qkv_norm_store(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, k_dim: int, v_dim: int, cache: torch.Tensor,
                   slots: Optional[torch.Tensor], qk_norm: int = QK_NORM_NONE, q_weight: Optional[torch.Tensor] = None,
                   k_weight: Optional[torch.Tensor] = None, qk_eps: float = 0.0, values_from_keys: bool = False,
                   value_norm_eps: Optional[float] = None, v_first: Optional[torch.Tensor] = None,
                   v_blend: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None,
                   inv_freq: Optional[torch.Tensor] = None, value_rows: bool = False) -> torch.Tensor:
    """From the projected rows qkv [T, Hq k_dim + Hkv k_dim (+ Hkv v_dim)] to q [T, Hq, Dc] and the cache
    [pages, 2, Hkv, P, Dc] (zeros beyond a head's own numbers): q and k normed per head (weights [k_dim]) or
    over the whole projection (weights [Hq k_dim] and [Hkv k_dim]), the values their own projection or the keys
    as projected (``values_from_keys``), each value head divided by its root mean square (``value_norm_eps``),
    then either left in ``v_first`` (float32 [T, Hkv v_dim]; ``v_blend`` None) for later layers or blended with
    it, v <- (1 - v_blend) v + v_blend v_first; the first 2 len(inv_freq) numbers of every q and k head rotated in
    half-split pairs by positions * inv_freq; k and v written at ``slots`` (page * P + offset; negative: nowhere),
    value tiles transposed ([Dc][P]) or, with ``value_rows``, as rows ([P][Dc])."""
    lib = load_library()
    _need(qkv, "qkv", _ACT, (None, None))
    T, dev = qkv.shape[0], qkv.device
    Hq, Hkv, Dk, Dv = int(num_heads), int(num_kv_heads), int(k_dim), int(v_dim)
    need = Hq * Dk + Hkv * Dk + (0 if values_from_keys else Hkv * Dv)
    if qkv.shape[1] < need:          # (rows may go on behind q | k | v: other outputs of the same product)
        raise KernelError(f"qkv_norm_store: rows of {qkv.shape[1]} numbers, {need} expected")
    _need(cache, "cache", qkv.dtype, (None, 2, Hkv, None, None), dev)
    P, Dc = cache.shape[3], cache.shape[4]
    if qk_norm != QK_NORM_NONE:
        n = (Hq * Dk, Hkv * Dk) if qk_norm == QK_NORM_WHOLE else (Dk, Dk)
        _need(q_weight, "q_weight", torch.float32, (n[0],), dev)
        _need(k_weight, "k_weight", torch.float32, (n[1],), dev)
    if slots is not None:
        _need(slots, "slots", torch.int32, (T,), dev)
    if v_first is not None:
        _need(v_first, "v_first", torch.float32, (T, Hkv * Dv), dev)
        if v_blend is not None:
            _need(v_blend, "v_blend", torch.float32, (1,), dev)
    elif v_blend is not None:
        raise KernelError("qkv_norm_store: a blend without the values to blend with")
    rot = 0
    if inv_freq is not None:
        _need(inv_freq, "inv_freq", torch.float32, (None,), dev)
        _need(positions, "positions", torch.int32, (T,), dev)
        rot = 2 * inv_freq.shape[0]
    q = torch.empty((T, Hq, Dc), dtype=qkv.dtype, device=dev)
    _check(lib.qe_qkv_norm_store(qkv.data_ptr(), qkv.shape[1], _ptr(q_weight), _ptr(k_weight), int(qk_norm), float(qk_eps),
                                 int(bool(values_from_keys)), int(value_norm_eps is not None),
                                 float(value_norm_eps or 0.0), _ptr(v_blend), _ptr(v_first),
                                 int(v_first is not None and v_blend is None), _ptr(positions), _ptr(inv_freq), rot,
                                 _ptr(slots), q.data_ptr(), cache.data_ptr(), T, Hq, Hkv, Dk, Dv, Dc, P,
                                 int(bool(value_rows)), _DT[qkv.dtype], _stream()), "qkv_norm_store")
    return q


def attention_talk(q: torch.Tensor, cache: torch.Tensor, positions: torch.Tensor, tok_seq: torch.Tensor,
                   block_table: torch.Tensor, scale: float, k_dim: int, v_dim: int, window: int = 0, chunk: int = 0,
                   bias: Optional[torch.Tensor] = None, talk: Optional[torch.Tensor] = None,
                   out: Optional[torch.Tensor] = None, out_scale: float = 1.0,
                   tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention whose scores get a bias by distance (``bias`` float32 [rows, Hq]: row min(i - j, rows - 1)) and are
    then mixed across heads (``talk`` float32 [Hq, Hq]: s'_h = sum_g talk[h, g] s_g) before the softmax.  q
    [T, Hq, Dc]; cache [pages, 2, Hkv, P, Dc] with keys and values both as rows; a head's keys have k_dim numbers,
    its values v_dim.  ``window`` / ``chunk`` as for attention().  out [T, Hq * v_dim] (may be a slice of columns
    of a wider tensor), multiplied by out_scale."""
    lib = load_library()
    _need(q, "q", _ACT, (None, None, None))
    T, Hq, Dc = q.shape
    dev = q.device
    _need(cache, "cache", q.dtype, (None, 2, None, None, Dc), dev)
    Hkv, P = cache.shape[2], cache.shape[3]
    _need(positions, "positions", torch.int32, (T,), dev)
    _need(tok_seq, "tok_seq", torch.int32, (T,), dev)
    _need(block_table, "block_table", torch.int32, (None, None), dev)
    if chunk:
        if window or chunk < 0:
            raise KernelError("attention_talk: chunks go without a window")
        window = -int(chunk)
    rows = 0
    if bias is not None:
        _need(bias, "bias", torch.float32, (None, Hq), dev)
        rows = bias.shape[0]
    if talk is not None:
        _need(talk, "talk", torch.float32, (Hq, Hq), dev)
    n = Hq * int(v_dim)
    if out is None:
        out = torch.empty((T, n), dtype=q.dtype, device=dev)
    if out.dtype != q.dtype or out.dim() != 2 or out.shape != (T, n) or out.stride(1) != 1 or out.device != dev:
        raise KernelError(f"attention_talk: out is {tuple(out.shape)} {out.dtype}, expected {(T, n)} {q.dtype}")
    n_tok = T
    if tokens is not None:
        _need(tokens, "tokens", torch.int32, (None,), dev)
        n_tok = tokens.shape[0]
    # a token's keys are dealt to several blocks while the tokens alone do not fill the machine
    splits = lib.qe_attention_talk_splits(n_tok, -int(window) if window < 0 else int(window))
    ws = None
    if splits > 1:
        ws = torch.empty((n_tok * splits * (2 * Hq + n),), dtype=torch.float32, device=dev)
    _check(lib.qe_attention_talk(q.data_ptr(), out.data_ptr(), out.stride(0) if T > 1 else n, float(out_scale),
                                 cache.data_ptr(), positions.data_ptr(), tok_seq.data_ptr(), block_table.data_ptr(),
                                 block_table.shape[1], _ptr(tokens), n_tok, _ptr(bias), rows, _ptr(talk), Hq, Hkv,
                                 int(k_dim), int(v_dim), Dc, P, float(scale), int(window), int(splits), _ptr(ws),
                                 _DT[q.dtype], _stream()),
           "attention_talk")
    return out


# ---- mixers with a matrix per head as their state -----------------------------------------------------------------------
def token_shift(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, tok_seq: torch.Tensor,
                single_rows: bool = False) -> torch.Tensor:
    """y[s] = x + (x' - x) * mu[s], x' the row of the token before in the same request (rows of a request are
    consecutive; tok_seq names its state row): x [T, W], mu float32 [n, W] -> [n, T, W].  What lies before a request's
    rows in this step is state[tok_seq[t], :W] (float32; zeros for a new request), which then takes the request's
    last row.  ``single_rows``: no two rows belong to one request (one launch instead of two)."""
    lib = load_library()
    _need(x, "x", _ACT, (None, None))
    T, W = x.shape
    _need(mu, "mu", torch.float32, (None, W), x.device)
    _need(tok_seq, "tok_seq", torch.int32, (T,), x.device)
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] < W or state.stride(1) != 1:
        raise KernelError("token_shift: the state is float32 [slots, >= W]")
    y = torch.empty((mu.shape[0], T, W), dtype=x.dtype, device=x.device)
    _check(lib.qe_token_shift(x.data_ptr(), mu.data_ptr(), mu.shape[0], state.data_ptr(), state.stride(0),
                              tok_seq.data_ptr(), y.data_ptr(), T, W, int(bool(single_rows)), _DT[x.dtype], _stream()),
           "token_shift")
    return y


def _rows_view(t: torch.Tensor, name: str, n: int, T: int):
    if t.dim() != 2 or t.shape != (T, n) or t.stride(1) != 1:
        raise KernelError(f"{name} is {tuple(t.shape)} with strides {t.stride()}, expected rows of {n} numbers")
    return t.stride(0) if T > 1 else n


def recurrence_chunk_len(head_dim: int) -> int:
    """Rows of a chunk of the chunked recurrence for heads of this many key channels."""
    return load_library().qe_recurrence_chunk_len(int(head_dim))


def recurrence_chunks(portions, chunk_len: int):
    """For portions given as (first row, rows) on the host: the ``chunks`` of linear_recurrence(), a pair of int32
    tensors (on the host) [n, 2] = (first row, rows <= chunk_len) and [m, 3] = (first chunk, chunks, first row)."""
    chunks, ports = [], []
    for start, n in portions:
        if n <= 0:
            continue
        ports.append((len(chunks), -(-n // chunk_len), start))
        chunks += [(start + r, min(chunk_len, n - r)) for r in range(0, n, chunk_len)]
    return (torch.tensor(chunks, dtype=torch.int32).view(-1, 2), torch.tensor(ports, dtype=torch.int32).view(-1, 3))


def linear_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor, tok_seq: torch.Tensor,
                      heads: int, decay: Optional[torch.Tensor] = None, decay_x: Optional[torch.Tensor] = None,
                      decay_bias: Optional[torch.Tensor] = None, bonus: Optional[torch.Tensor] = None,
                      silu: bool = False, chunks=None) -> torch.Tensor:
    """Per head, with a 32-bit state S [D][Dv] per request (state[tok_seq[t]], float32 [slots, >= H D Dv]):
    with ``decay`` (float32 [H]):  S <- decay_h S + k_t v_t^T, o_t = S^T q_t;
    with ``decay_x`` float32 [T, H D], ``decay_bias`` and ``bonus`` (float32 [H D]):  o_t = (S + diag(bonus) k_t v_t^T)^T q_t,
    then S <- diag(w_t) S + k_t v_t^T with w_t = exp(-exp(decay_x_t + decay_bias)).
    q, k [T, H D], v [T, H Dv] (column slices of one wider tensor are taken as they are, all with one row stride);
    ``silu``: the three pass silu first.  Returns o float32 [T, H, Dv].
    ``chunks`` (recurrence_chunks() of all rows' portions, on the device, for recurrence_chunk_len(D)): the rows are
    taken chunk by chunk, the chunks in parallel, instead of row by row: for long portions."""
    lib = load_library()
    T, dev, H = q.shape[0], q.device, int(heads)
    if q.dtype not in _ACT or k.dtype != q.dtype or v.dtype != q.dtype:
        raise KernelError("linear_recurrence: q, k and v of one element type")
    D, Dv = q.shape[1] // H, v.shape[1] // H
    sq, sk, sv = _rows_view(q, "q", H * D, T), _rows_view(k, "k", H * D, T), _rows_view(v, "v", H * Dv, T)
    if T > 1 and not sq == sk == sv:
        raise KernelError("linear_recurrence: q, k and v with different row strides")
    _need(tok_seq, "tok_seq", torch.int32, (T,), dev)
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] < H * D * Dv or state.stride(1) != 1:
        raise KernelError("linear_recurrence: the state is float32 [slots, >= H D Dv]")
    mode, sw = 0, 0
    if decay is not None:
        _need(decay, "decay", torch.float32, (H,), dev)
    else:
        mode = 1
        if decay_x is None or decay_x.dtype != torch.float32:
            raise KernelError("linear_recurrence: no decays")
        sw = _rows_view(decay_x, "decay_x", H * D, T)
        _need(decay_bias, "decay_bias", torch.float32, (H * D,), dev)
        _need(bonus, "bonus", torch.float32, (H * D,), dev)
    out = torch.empty((T, H, Dv), dtype=torch.float32, device=dev)
    if chunks is not None and chunks[0].shape[0]:
        ch, po = chunks
        _need(ch, "chunks", torch.int32, (None, 2), dev)
        _need(po, "portions", torch.int32, (None, 3), dev)
        ws = torch.empty((ch.shape[0] * H * (D * Dv + D),), dtype=torch.float32, device=dev)
        _check(lib.qe_linear_recurrence_chunked(q.data_ptr(), k.data_ptr(), v.data_ptr(), sq, _ptr(decay_x), sw,
                                                _ptr(decay_bias), _ptr(bonus), _ptr(decay), mode, int(bool(silu)),
                                                state.data_ptr(), state.stride(0), tok_seq.data_ptr(), ch.data_ptr(),
                                                ch.shape[0], po.data_ptr(), po.shape[0], ws.data_ptr(), out.data_ptr(),
                                                H, D, Dv, _DT[q.dtype], _stream()), "linear_recurrence (chunked)")
        return out
    _check(lib.qe_linear_recurrence(q.data_ptr(), k.data_ptr(), v.data_ptr(), sq, _ptr(decay_x), sw, _ptr(decay_bias),
                                    _ptr(bonus), _ptr(decay), mode, int(bool(silu)), state.data_ptr(), state.stride(0),
                                    tok_seq.data_ptr(), out.data_ptr(), T, H, D, Dv, _DT[q.dtype], _stream()),
           "linear_recurrence")
    return out


GATE_NONE, GATE_SILU, GATE_SIGMOID = 0, 1, 2


def gated_norm(o: torch.Tensor, weight: torch.Tensor, eps: float, groups: int, out_dtype: torch.dtype,
               gate: Optional[torch.Tensor] = None, gate_act: int = GATE_NONE, scale: float = 1.0,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = o / rms(o) * weight * act(gate) * scale per row of o (float32 [T, N]), the root mean square taken over
    each of ``groups`` equal pieces of the row; gate [T, N] (may be a slice of columns), act silu or sigmoid."""
    lib = load_library()
    _need(o, "o", torch.float32, (None, None))
    T, N = o.shape
    _need(weight, "weight", torch.float32, (N,), o.device)
    sg, dg = 0, F32
    if gate is not None:
        sg, dg = _rows_view(gate, "gate", N, T), _DT[gate.dtype]
    if out is None:
        out = torch.empty((T, N), dtype=out_dtype, device=o.device)
    so = _rows_view(out, "out", N, T)
    _check(lib.qe_gated_norm(o.data_ptr(), weight.data_ptr(), _ptr(gate), sg, dg, int(gate_act), float(eps), float(scale),
                             out.data_ptr(), so, _DT[out.dtype], T, N, int(groups), _stream()), "gated_norm")
    return out


UNARY_GELU, UNARY_TANH, UNARY_SOFTCAP = 0, 1, 2


def unary(z: torch.Tensor, kind: int, out_dtype: Optional[torch.dtype] = None, cap: float = 0.0,
          inplace: bool = False) -> torch.Tensor:
    """Element by element in 32-bit: the exact gelu 0.5 z (1 + erf(z / sqrt 2)), tanh, or cap * tanh(z / cap)."""
    lib = load_library()
    if not z.is_contiguous() or z.dtype not in _ACT:
        raise KernelError("unary: a contiguous float32 or bfloat16 tensor")
    y = z if inplace else torch.empty(z.shape, dtype=out_dtype or z.dtype, device=z.device)
    _check(lib.qe_unary(z.data_ptr(), _DT[z.dtype], y.data_ptr(), _DT[y.dtype], z.numel(), int(kind), float(cap),
                        _stream()), "unary")
    return y


def scaled_sum(a: torch.Tensor, sa: float, b: torch.Tensor, sb: float) -> torch.Tensor:
    """sa * a + sb * b in 32-bit, float32."""
    lib = load_library()
    if a.shape != b.shape or a.dtype != b.dtype or a.dtype not in _ACT or not a.is_contiguous() or not b.is_contiguous():
        raise KernelError("scaled_sum: two contiguous tensors of one shape and type")
    y = torch.empty(a.shape, dtype=torch.float32, device=a.device)
    _check(lib.qe_scaled_sum(a.data_ptr(), float(sa), b.data_ptr(), float(sb), _DT[a.dtype], y.data_ptr(), a.numel(),
                             _stream()), "scaled_sum")
    return y


def moe_row_gate(dst: torch.Tensor, src: torch.Tensor, gate_logits: torch.Tensor, accumulate: bool) -> None:
    """dst[t] (+)= sigmoid(gate_logits[t]) * src[t]: dst float32 [T, H], src [T, H] (may be dst itself), gate_logits
    float32 [T] or a column of wider rows.  An expert that every token uses, weighed by one number a token."""
    lib = load_library()
    _need(dst, "dst", torch.float32, (None, None))
    T, H = dst.shape
    _need(src, "src", _ACT, (T, H), dst.device)
    if gate_logits.dtype != torch.float32 or gate_logits.dim() != 1 or gate_logits.shape[0] != T or not gate_logits.is_cuda:
        raise KernelError("moe_row_gate: one 32-bit gate a row")
    _check(lib.qe_moe_row_gate(dst.data_ptr(), src.data_ptr(), _DT[src.dtype], gate_logits.data_ptr(),
                               max(1, gate_logits.stride(0)), T, H, int(bool(accumulate)), _stream()), "moe_row_gate")


def diff_heads(a: torch.Tensor, num_heads: int, num_kv_heads: int, v_dim: int, lam: float, eps: float, out_scale: float,
               gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Joins the two maps of differential attention: a [T, 2 H, Dc], map m of head h = g (H / G) + j at query head
    g (2 H / G) + m (H / G) + j -> out [T, H, v_dim]: o = a1 - lam a2, divided by its root mean square over v_dim
    (eps inside the root), times out_scale, times sigmoid(gate[t, h]) (gate [T, H], or H columns of wider rows)."""
    lib = load_library()
    _need(a, "a", _ACT, (None, 2 * int(num_heads), None))
    T, _, Dc = a.shape
    H, G, Dv = int(num_heads), int(num_kv_heads), int(v_dim)
    gs = 0
    if gate is not None:
        if gate.dim() != 2 or gate.shape != (T, H) or gate.stride(1) != 1 or gate.dtype != a.dtype or gate.device != a.device:
            raise KernelError("diff_heads: one gate a head, in the rows' element type")
        gs = gate.stride(0)
    out = torch.empty((T, H, Dv), dtype=a.dtype, device=a.device)
    _check(lib.qe_diff_heads(a.data_ptr(), out.data_ptr(), _ptr(gate), gs, T, H, G, Dv, Dc, float(lam), float(eps),
                             float(out_scale), _DT[a.dtype], _stream()), "diff_heads")
    return out
