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
        "qe_rmsnorm": [vp, vp, i32, i32, i64, vp, vp, vp, i32, i32, f32, i32, vp],
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
        "qe_attention_prefill_run": [vp, vp, vp, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, f32, i32, i32, i32, i32,
                                     i32, vp, i64, vp],
        "qe_attention_prefill_plan_segments": [i32, i32, i32],
        "qe_attention_prefill_tiles_run": [vp, i32, i32, vp, i32, vp],
        "qe_attention_prefill_workspace_bytes_for": [i32, i32, i32, i32, i32],
        "qe_attention_prefill_plan": [i32, i32, i32, i32],
        "qe_attention_prefill_plan_uncut_keys": [],
        "qe_attention_prefill_workspace_bytes": [i32, i32, i32, i32, i32, i32],
        "qe_attention_decode_run": [vp, vp, vp, vp, i32, vp, vp, vp, i32, vp, i32, i32, i32, i32, f32, i32, i32, i32, vp, i64, vp],
        "qe_attention_decode_fused_run": [vp, vp, vp, vp, i32, vp, vp, vp, i32, vp, vp, vp, vp, f32, vp,
                                          i32, i32, i32, i32, f32, i32, i32, i32, vp, i64, vp],
        "qe_qk_rope_store": [vp, vp, vp, vp, f32, vp, i32, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, vp],
        "qe_qk_rope_store_parts": [vp, i32, vp, vp, vp, vp, f32, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, vp],
        "qe_qk_rope_store_parts_supported": [i32, i32],
        "qe_gemm_partial_preferred": [i32, i32, i32, i32, i32],
        "qe_gemm_branch_splits": [i32, i32, i32, i32, i32],
        "qe_attention": [vp, vp, vp, vp, vp, vp, i32, vp, i32, i32, i32, i32, i32, f32, i32, i32, vp],
        "qe_argmax": [vp, vp, i32, i32, vp, i64, vp],
        "qe_argmax_static": [vp, vp, i32, i32, vp],
        "qe_sample": [vp, vp, vp, vp, i32, i32, vp],
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
            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm of the 32-bit stream h [T, H] into out_dtype.

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
                          out.data_ptr(), n, H, float(eps), _DT[out_dtype], _stream()), "rmsnorm")
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
              other_keys_row: Optional[int] = None, shared_keys: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [T, Hq, D]; cache [pages, 2, Hkv, P, D] (key tiles [P][D], value tiles transposed [D][P]);
    positions, tok_seq int32 [T]; block_table int32 [B, max_blocks].  Token t sees the keys at
    positions max(0, p - window + 1) .. p of request tok_seq[t] (window 0: all).  The caller
    guarantees that those positions have pages in the table.

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

    def generic(tokens):
        n = T if tokens is None else tokens.shape[0]
        _check(lib.qe_attention(q.data_ptr(), out.data_ptr(), cache.data_ptr(), positions.data_ptr(),
                                tok_seq.data_ptr(), block_table.data_ptr(), max_blocks, _ptr(tokens), n,
                                Hq, Hkv, D, P, float(scale), int(window), _DT[q.dtype], _stream()), "attention")

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
                                               D, P, float(scale), int(window), int(max_dec_position),
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
                                                max_blocks, Hq, Hkv, D, P, float(scale), int(window),
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
