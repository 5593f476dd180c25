"""Python bindings of the HIP library: one function per kernel entry point.

Each wrapper checks on the host that operand shapes, dtypes and devices match what its kernel
assumes, then calls the C function on torch's current HIP stream.  There is no other
implementation behind these functions: without the library, or without a GPU, they raise.
"""
from __future__ import annotations

import ctypes
import os
import threading
from typing import Optional

import torch

from ..csrc import build as _build

EPI_NONE, EPI_GEGLU, EPI_SOFTCAP = 0, 1, 2
LAYOUT_ROW, LAYOUT_FRAG16 = 0, 1
LINEAR_AUTO, LINEAR_GENERIC, LINEAR_SKINNY, LINEAR_MFMA, LINEAR_TILED_W16, LINEAR_TILED_W32 = 0, 1, 2, 3, 4, 5
ABI_VERSION = 12
GATED_SILU = -1.0        # epi_param of EPI_GEGLU that picks silu(gate) * up
UNARY_RELU2 = -1.0       # epi_param of EPI_SOFTCAP that picks the square of max(y, 0) instead of the capped form

_lib = None
_lib_path = None
_lock = threading.Lock()


class HipLibraryError(RuntimeError):
    """The HIP library is missing, cannot be built or loaded, or a kernel refused its arguments."""


def _declare(lib) -> None:
    c = ctypes
    P, I, L, F = c.c_void_p, c.c_int, c.c_long, c.c_float
    lib.alice_last_error.restype = c.c_char_p
    lib.alice_abi_version.restype = I
    lib.alice_device_arch.argtypes = [c.c_char_p, I]
    sigs = {
        "alice_embed": [P, P, I, I, P, I, I, I, F, P],
        "alice_add_norm": [P, P, I, L, P, P, I, P, I, P, I, I, F, F, F, F, I, I, P],
        "alice_softcap": [P, L, F, I, P],
        "alice_add_branches": [P, I, P, P, P, P, I, P, P, P, I, I, I, I, P],
        "alice_linear": [P, I, P, I, I, P, I, I, I, I, I, F, I, I, I, I, I, P],
        "alice_linear_split_hint": [I, I, I, I],
        "alice_to_frag16": [P, P, I, I, P],
        "alice_frag16_supported": [I, I, I],
        "alice_rope_cache_write": [P, I, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I, I, I, I, P],
        "alice_mlstm_step": [P, I, P, P, P, I, P, I, P, P, P, P, P, I, I, I, I, I, F, F, P],
        "alice_mlstm_chunks": [P, I, P, P, P, I, P, I, P, P, P, P, P, P, I, I, I, I, I, I, F, F, I, P],
        "alice_mlstm_chunks_supported": [I, I, I, I],
        "alice_mlstm_cols": [P, I, P, P, P, I, P, I, P, P, P, P, P, P, I, I, I, I, I, I, F, F, P],
        "alice_gelu_mul_rows": [P, I, P, I, I, I, P, P, I, I, I, I, I, P],
        "alice_linear_rope_cache": [P, I, P, I, I, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, P],
        "alice_attention_mfma_supported": [I],
        "alice_attention_prefill": [P, P, P, P, P, P, P, I, I, I, I, I, I, I, F, F, I, I, I, P],
        "alice_attention_decode": [P, P, P, P, P, P, P, I, I, I, I, I, I, F, F, I, I, I, P, I, P],
        "alice_attention_generic": [P, I, P, P, P, P, P, P, I, I, I, I, I, I, F, F, I, P, I, I, P, I, P],
        "alice_head_gate": [P, I, P, I, I, I, I, P],
        "alice_attention_masked": [P, I, P, P, P, P, P, P, I, I, I, I, I, I, F, F, I, P, I, I, P, I, I, F, I, I, P, P, P, P, P],
        "alice_attention_tiled": [P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, F, I, I, I, P, P, P, P, P, I, I, F, I, P],
        "alice_attention_tiled_supported": [I, I],
        "alice_attention_split": [P, I, P, P, P, P, P, P, P, I, I, I, I, I, I, I, F, I, I, I, I, P, P, P, P, P, I, I, F, P, P],
        "alice_attention_split_supported": [I, I, I, I, I],
        "alice_attention_split_runs": [I],
        "alice_mix_heads": [P, P, P, I, F, P, I, I, I, I, I, I, P],
        "alice_qkv_prepare": [P, I, I, P, P, P, P, I, P, P, I, I, P, P, P, P, P, I, I, I, I, I, I, I, I, P, F, P, P],
        "alice_short_conv": [P, I, I, I, I, P, P, P, P, I, P, P, P, I, I, P],
        "alice_ssm_prepare": [P, I, I, P, P, P, P, I, I, P],
        "alice_delta_prepare": [P, I, I, I, I, F, F, P, P, P, P, I, I, P, I, I, P],
        "alice_matrix_recurrence": [P, I, I, P, I, I, P, I, I, P, I, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P],
        "alice_matrix_recurrence_columns": [I, I, I, I],
        "alice_norm_gate": [P, I, I, P, I, I, I, P, I, F, P, I, I, P],
        "alice_route_topk": [P, P, P, I, I, I, P],
        "alice_scale_columns": [P, I, P, P, I, I, I, I, P],
        "alice_expert_products": [P, P, P, P, P, P, P, P, I, I, I, I, I, F, P],
        "alice_add_rows": [P, P, P, I, I, P],
        "alice_latent_prepare": [P, I, I, I, I, P, P, F, P, P, P, P, P, I, I, I, P, P, I, I, P],
        "alice_heads_linear": [P, I, L, I, P, I, P, I, L, I, I, I, I, I, I, P, P, P, P],
        "alice_heads_linear_mfma_supported": [I, I, I],
        "alice_heads_linear_mfma": [P, L, I, P, P, L, I, I, I, I, I, I, P, P, P, P],
        "alice_latent_attention": [P, I, P, P, P, P, P, I, I, I, I, I, I, F, I, I, P],
        "alice_latent_tiled_supported": [I, I],
        "alice_latent_tiled_max_splits": [],
        "alice_latent_tiled": [P, P, P, P, P, P, P, I, I, I, I, I, I, I, F, I, I, I, P],
        "alice_gla": [P, I, I, I, I, I, P, P, F, F, F, P, I, F, P, I, P, P, P, P, I, I, I, I, I, I, I, P],
        "alice_linear_parts_split": [I, I, I, I, I],
        "alice_linear_parts": [P, I, I, I, P, P, I, I, P],
        "alice_argmax": [P, P, P, P, I, I, P],
        "alice_argmax_chunks": [I, I],
        "alice_sample_workspace": [I, I],
        "alice_sample": [P, P, P, P, I, I, F, I, F, P],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = I
    lib.alice_attention_decode_workspace.argtypes = [I, I, I, I]
    lib.alice_attention_decode_workspace.restype = L
    lib.alice_attention_split_workspace.argtypes = [I, I, I, I, I, I]
    lib.alice_attention_split_workspace.restype = L
    lib.alice_mlstm_chunks_workspace.argtypes = [I, I, I, I, I, I]
    lib.alice_mlstm_chunks_workspace.restype = L
    lib.alice_expert_rows.argtypes = [I, I, I]
    lib.alice_expert_rows.restype = L


def _open(path: str):
    try:
        return ctypes.CDLL(path)
    except OSError as e:
        raise HipLibraryError(f"cannot load {path}: {e}") from e


def _built_from_these_sources(lib) -> bool:
    try:
        fn = lib.alice_source_digest
    except AttributeError:
        return False
    fn.restype = ctypes.c_char_p
    return fn().decode() == _build.source_digest()


def library():
    """The loaded HIP library: the built one if it was made from the sources beside these bindings, else
    built with hipcc at the first call."""
    global _lib, _lib_path
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        lib = path = None
        for cand in _build.built_libraries():
            found = _open(cand)
            if _built_from_these_sources(found):
                lib, path = found, cand
                break
            # a library left from other sources (an older checkout's, an edit after the last build) would give
            # results that belong to no version of the code: it is never used
            _build._say(f"{cand} was built from other sources than the ones beside it")
        if lib is None:
            try:
                path = _build.build(verbose=True)
            except Exception as e:
                raise HipLibraryError(f"the HIP library is not built and building it failed: {e}") from e
            lib = _open(path)
        _declare(lib)
        if lib.alice_abi_version() != ABI_VERSION:
            raise HipLibraryError(f"{path} has interface version {lib.alice_abi_version()}, these bindings "
                                  f"need {ABI_VERSION}: rebuild it (python -m alice_llm_amd.csrc.build)")
        _lib, _lib_path = lib, path
        return _lib


def library_ready() -> bool:
    """Whether kernels can run at all here (a GPU is visible); skeleton models built on the CPU to list
    their tensors do not touch the library."""
    return torch.cuda.is_available()


def library_path() -> Optional[str]:
    """The library in use, or the one that would be tried first."""
    return _lib_path or _build.find_library()


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise HipLibraryError("no GPU is visible to torch: this library runs on an MI355X (gfx950) only "
                              "and has no CPU path")
    return torch.device("cuda", torch.cuda.current_device())


def _call(name: str, *args) -> None:
    lib = library()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise HipLibraryError(f"{name}: {lib.alice_last_error().decode()}")


def _stream() -> int:
    # torch's current stream of the current device, as the raw handle: the same value as
    # torch.cuda.current_stream().cuda_stream without building a Stream object for every launch
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return 0
    if dt == torch.bfloat16:
        return 1
    raise HipLibraryError(f"dtype {dt} has no kernel: float32 and bfloat16 only")


def _dev(t: torch.Tensor, name: str, dtype=None, shape=None) -> int:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise HipLibraryError(f"{name} must be a GPU tensor")
    if not t.is_contiguous():
        raise HipLibraryError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise HipLibraryError(f"{name} must be {dtype}, found {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise HipLibraryError(f"{name} must have shape {tuple(shape)}, found {tuple(t.shape)}")
    return t.data_ptr()


def _opt(t, name, dtype=None, shape=None) -> Optional[int]:
    return None if t is None else _dev(t, name, dtype, shape)


# ------------------------------------------------------------------------------------ ops

def embed(tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float,
          vocab: int, dim: int, layout: int = LAYOUT_ROW) -> None:
    T = tokens.numel()
    _dev(tokens, "tokens", torch.int32)
    _dev(out, "out", torch.float32, (T, dim))
    if layout == LAYOUT_ROW:
        _dev(table, "table", None, (vocab, dim))
    else:
        _dev(table, "table", torch.bfloat16)
        need = ((vocab + 15) // 16 * 16) * ((dim + 31) // 32 * 32)
        if table.numel() != need:
            raise HipLibraryError(f"table in fragment layout must hold {need} elements, found {table.numel()}")
    _call("alice_embed", tokens.data_ptr(), table.data_ptr(), dtype_code(table.dtype), layout,
          out.data_ptr(), T, dim, vocab, float(scale), _stream())


def add_norm(resid: torch.Tensor, branch: Optional[torch.Tensor], w_post: Optional[torch.Tensor],
             w_pre: Optional[torch.Tensor], out: Optional[torch.Tensor], *, eps_post: float = 0.0,
             eps_pre: float = 0.0, off_post: float = 0.0, off_pre: float = 0.0,
             rows: Optional[torch.Tensor] = None, n_partials: int = 1, full_precision: bool,
             out_layout: int = LAYOUT_ROW) -> None:
    """resid += norm_post(sum of branch partials); out = norm_pre(resid).  Each piece is optional.
    out_layout FRAG16: `out` is a flat bfloat16 buffer of ceil16(T) * H elements in fragment order."""
    if resid.dim() != 2:
        raise HipLibraryError("resid must be [T, H]")
    Tres, H = resid.shape
    _dev(resid, "resid", torch.float32)
    T = Tres if rows is None else rows.numel()
    stride = 0
    if branch is not None:
        want = (n_partials, Tres, H) if n_partials > 1 else (Tres, H)
        _dev(branch, "branch", torch.float32, want)
        stride = Tres * H
    elif n_partials != 1:
        raise HipLibraryError("partial sums need a branch")
    w_dtype = None
    for w, nm in ((w_post, "w_post"), (w_pre, "w_pre")):
        if w is not None:
            _dev(w, nm, None, (H,))
            if w_dtype is not None and w.dtype != w_dtype:
                raise HipLibraryError("w_post and w_pre must have one dtype")
            w_dtype = w.dtype
    if w_post is not None and branch is None:
        raise HipLibraryError("w_post without a branch")
    if out is not None and out_layout == LAYOUT_FRAG16:
        _dev(out, "out", torch.bfloat16, (frag_rows(T) * H,))
    elif out is not None:
        _dev(out, "out", None, (T, H))
    elif w_pre is not None:
        raise HipLibraryError("w_pre without an output")
    if rows is not None:
        _dev(rows, "rows", torch.int32)
    _call("alice_add_norm", resid.data_ptr(), _opt(branch, "branch"), n_partials, stride,
          _opt(w_post, "w_post"), _opt(w_pre, "w_pre"), dtype_code(w_dtype or torch.float32),
          _opt(out, "out"), dtype_code(out.dtype if out is not None else torch.float32),
          _opt(rows, "rows"), T, H, float(eps_post), float(eps_pre), float(off_post), float(off_pre),
          int(full_precision), int(out_layout), _stream())


MAX_BRANCHES = 4
ADD_BRANCHES_MAX_WIDTH = 8192      # rows that add_branches holds in registers


def add_branches(resid: torch.Tensor, branches, out: Optional[torch.Tensor] = None, *, full_precision: bool) -> None:
    """resid += sum of norm_j(branch_j) in one kernel.  branches: up to four (tensor, weight, eps, offset) with tensor
    float32 [T, H] or [S, T, H] partial results; weight None adds the branch as it is, else it is RMS-normed over
    the row first and multiplied by (offset + weight).  out (optional): the new rows in its own dtype, [T, H]."""
    T, H = resid.shape
    _dev(resid, "resid", torch.float32)
    n = len(branches)
    if not 1 <= n <= MAX_BRANCHES:
        raise HipLibraryError(f"add_branches takes 1 to {MAX_BRANCHES} branches, found {n}")
    c = ctypes
    ptrs, parts, strides, ws, eps, offs = (c.c_void_p * n)(), (c.c_int * n)(), (c.c_long * n)(), (c.c_void_p * n)(), (c.c_float * n)(), (c.c_float * n)()
    w_dtype = None
    for j, (b, w, e, o) in enumerate(branches):
        p = b.shape[0] if b.dim() == 3 else 1
        _dev(b, "branch", torch.float32, (p, T, H) if b.dim() == 3 else (T, H))
        ptrs[j], parts[j], strides[j] = b.data_ptr(), p, T * H
        if w is not None:
            _dev(w, "weight", None, (H,))
            if w_dtype is not None and w.dtype != w_dtype:
                raise HipLibraryError("the branches' norm weights must have one dtype")
            w_dtype = w.dtype
        ws[j], eps[j], offs[j] = (None if w is None else w.data_ptr()), float(e), float(o)
    if out is not None:
        _dev(out, "out", None, (T, H))
    _call("alice_add_branches", resid.data_ptr(), n, ptrs, parts, strides, ws, dtype_code(w_dtype or torch.float32), eps, offs,
          _opt(out, "out"), dtype_code(out.dtype if out is not None else torch.float32), T, H, int(full_precision), _stream())


def frag_rows(rows: int) -> int:
    """Rows of an activation buffer in fragment order: padded to whole tiles of 16."""
    return -(-rows // 16) * 16


def softcap_(x: torch.Tensor, cap: float, full_precision: bool) -> None:
    _dev(x, "x", torch.float32)
    _call("alice_softcap", x.data_ptr(), x.numel(), float(cap), int(full_precision), _stream())


def linear(x: torch.Tensor, w: torch.Tensor, y: torch.Tensor, *, n_out: int, k_in: int,
           layout: int = LAYOUT_ROW, epilogue: int = EPI_NONE, epi_param: float = 0.0,
           split_k: int = 1, variant: int = LINEAR_AUTO, full_precision: bool, rows: Optional[int] = None,
           x_layout: int = LAYOUT_ROW, y_layout: int = LAYOUT_ROW) -> None:
    """y = x . W^T.  W: [n_out (2 n_out for GeGLU), k_in] row-major, or its fragment layout.
    x_layout / y_layout FRAG16: activations as flat bfloat16 buffers of ceil16(rows) * width elements in
    fragment order (then `rows` gives M)."""
    if x_layout == LAYOUT_FRAG16:
        if rows is None:
            raise HipLibraryError("activations in fragment order need the number of rows")
        M = rows
        _dev(x, "x", torch.bfloat16, (frag_rows(M) * k_in,))
    else:
        if x.dim() != 2 or x.shape[1] != k_in:
            raise HipLibraryError(f"x must be [M, {k_in}], found {tuple(x.shape)}")
        M = x.shape[0]
        _dev(x, "x")
    w_rows = n_out * (2 if epilogue == EPI_GEGLU else 1)
    if layout == LAYOUT_ROW:
        _dev(w, "w", None, (w_rows, k_in))
    else:
        _dev(w, "w", torch.bfloat16)
        need = ((w_rows + 15) // 16 * 16) * ((k_in + 31) // 32 * 32)
        if w.numel() != need:
            raise HipLibraryError(f"w in fragment layout must hold {need} elements, found {w.numel()}")
    if y_layout == LAYOUT_FRAG16:
        _dev(y, "y", torch.bfloat16, (frag_rows(M) * n_out,))
    else:
        want = (split_k, M, n_out) if split_k > 1 else (M, n_out)
        _dev(y, "y", None, want)
    if split_k > 1 and y.dtype != torch.float32:
        raise HipLibraryError("partial sums are float32")
    _call("alice_linear", x.data_ptr(), dtype_code(x.dtype), w.data_ptr(), dtype_code(w.dtype), layout,
          y.data_ptr(), dtype_code(y.dtype), M, n_out, k_in, epilogue, float(epi_param), split_k, variant,
          int(full_precision), int(x_layout), int(y_layout), _stream())


def linear_split_hint(M: int, N: int, K: int, layout: int) -> int:
    return library().alice_linear_split_hint(M, N, K, layout)


def to_frag16(w: torch.Tensor) -> torch.Tensor:
    """A row-major bfloat16 [N, K] matrix rearranged into the fragment layout (flat, zero padded)."""
    _dev(w, "w", torch.bfloat16)
    if w.dim() != 2:
        raise HipLibraryError("w must be [N, K]")
    N, K = w.shape
    out = torch.empty(((N + 15) // 16 * 16) * ((K + 31) // 32 * 32), dtype=torch.bfloat16, device=w.device)
    _call("alice_to_frag16", w.data_ptr(), out.data_ptr(), N, K, _stream())
    return out


def rope_cache_write(qkv: torch.Tensor, q_out: torch.Tensor, k_pool: Optional[torch.Tensor],
                     v_pool: Optional[torch.Tensor], cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                     positions: torch.Tensor, seq_of_token: Optional[torch.Tensor],
                     block_table: Optional[torch.Tensor], *, num_heads: int, num_kv_heads: int, head_dim: int,
                     rotary_dim: int, max_position: int, kv_layout: int = 0, interleaved: bool = False,
                     value_head_dim: Optional[int] = None) -> None:
    """Rotate q and k; write k and v at their positions into the pools [pages, nKV, page, d]
    (values [pages, nKV, page, value_head_dim] where that differs from d).
    With k_pool None the row holds q only (num_kv_heads = 0) and nothing is cached.
    `max_position` is the largest position among `positions` (the host knows it): checked against the tables.
    interleaved: the q and k heads of qkv hold the rotated pairs (j, j + d/2) at 2j and 2j + 1 (a projection
    with its rows in that order made them); the outputs are in the plain order either way."""
    T = qkv.shape[0]
    dt = qkv.dtype
    _dev(qkv, "qkv")
    row_width = qkv.shape[1]
    dv = head_dim if value_head_dim is None else int(value_head_dim)
    if qkv.dim() != 2 or row_width < num_heads * head_dim + (num_kv_heads * (head_dim + dv) if k_pool is not None else 0):
        raise HipLibraryError(f"qkv rows of {tuple(qkv.shape)} are too short for the heads")
    _dev(q_out, "q_out", dt, (T, num_heads * head_dim))
    _dev(positions, "positions", torch.int32, (T,))
    if cos is not None:
        if cos.dim() != 2 or cos.shape[1] != rotary_dim // 2 or sin.shape != cos.shape:
            raise HipLibraryError(f"cos/sin tables must be [positions, {rotary_dim // 2}]")
        _dev(cos, "cos", torch.float32)
        _dev(sin, "sin", torch.float32)
        if max_position >= cos.shape[0]:
            raise HipLibraryError(f"position {max_position} is beyond the rotation tables ({cos.shape[0]} positions)")
    page_size = n_pages = bt_stride = 0
    if k_pool is not None:
        if k_pool.dim() != 4 or k_pool.shape[1] != num_kv_heads or k_pool.shape[3] != head_dim:
            raise HipLibraryError(f"k_pool must be [pages, {num_kv_heads}, page, {head_dim}], found {tuple(k_pool.shape)}")
        _dev(k_pool, "k_pool", dt)
        _dev(v_pool, "v_pool", dt, tuple(k_pool.shape[:3]) + (dv,))
        n_pages, _, page_size, _ = k_pool.shape
        _dev(seq_of_token, "seq_of_token", torch.int32, (T,))
        _dev(block_table, "block_table", torch.int32)
        if block_table.dim() != 2:
            raise HipLibraryError("block_table must be [sequences, pages per sequence]")
        bt_stride = block_table.shape[1]
        if max_position // page_size >= bt_stride:
            raise HipLibraryError(f"position {max_position} is beyond the block table ({bt_stride} pages of {page_size})")
    _call("alice_rope_cache_write", qkv.data_ptr(), dtype_code(dt), q_out.data_ptr(), _opt(k_pool, "k_pool"),
          _opt(v_pool, "v_pool"), _opt(cos, "cos"), _opt(sin, "sin"), positions.data_ptr(),
          _opt(seq_of_token, "seq_of_token"), _opt(block_table, "block_table"), bt_stride, T, row_width, num_heads,
          num_kv_heads, head_dim, rotary_dim, page_size, n_pages, int(kv_layout), int(interleaved), dv, _stream())


def linear_rope_cache(x: torch.Tensor, w: torch.Tensor, q_out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                      cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor, seq_of_token: torch.Tensor,
                      block_table: torch.Tensor, *, k_in: int, num_heads: int, num_kv_heads: int, head_dim: int,
                      max_position: int, kv_layout: int, rows: Optional[int] = None, x_layout: int = LAYOUT_ROW) -> None:
    """The fused q|k|v projection with the rotation and the cache write as its epilogue: what linear() followed by rope_cache_write(interleaved=True) gives.  w: the fragment layout of the
    [(nH + 2 nKV) d, k_in] matrix whose q and k heads have their rows in pair order."""
    if x_layout == LAYOUT_FRAG16:
        if rows is None:
            raise HipLibraryError("activations in fragment order need the number of rows")
        M = rows
        _dev(x, "x", torch.bfloat16, (frag_rows(M) * k_in,))
    else:
        if x.dim() != 2 or x.shape[1] != k_in:
            raise HipLibraryError(f"x must be [M, {k_in}], found {tuple(x.shape)}")
        M = x.shape[0]
        _dev(x, "x", torch.bfloat16)
    n_rows = (num_heads + 2 * num_kv_heads) * head_dim
    _dev(w, "w", torch.bfloat16)
    need = ((n_rows + 15) // 16 * 16) * ((k_in + 31) // 32 * 32)
    if w.numel() != need:
        raise HipLibraryError(f"w in fragment layout must hold {need} elements, found {w.numel()}")
    _dev(q_out, "q_out", torch.bfloat16, (M, num_heads * head_dim))
    if k_pool.dim() != 4 or k_pool.shape[1] != num_kv_heads or k_pool.shape[3] != head_dim:
        raise HipLibraryError(f"k_pool must be [pages, {num_kv_heads}, page, {head_dim}], found {tuple(k_pool.shape)}")
    _dev(k_pool, "k_pool", torch.bfloat16)
    _dev(v_pool, "v_pool", torch.bfloat16, k_pool.shape)
    n_pages, _, page_size, _ = k_pool.shape
    if cos.dim() != 2 or cos.shape[1] != head_dim // 2 or sin.shape != cos.shape:
        raise HipLibraryError(f"cos/sin tables must be [positions, {head_dim // 2}]")
    _dev(cos, "cos", torch.float32)
    _dev(sin, "sin", torch.float32)
    if max_position >= cos.shape[0]:
        raise HipLibraryError(f"position {max_position} is beyond the rotation tables ({cos.shape[0]} positions)")
    _dev(positions, "positions", torch.int32, (M,))
    _dev(seq_of_token, "seq_of_token", torch.int32, (M,))
    _dev(block_table, "block_table", torch.int32)
    if block_table.dim() != 2 or max_position // page_size >= block_table.shape[1]:
        raise HipLibraryError(f"position {max_position} is beyond the block table {tuple(block_table.shape)}")
    _call("alice_linear_rope_cache", x.data_ptr(), int(x_layout), w.data_ptr(), M, k_in, q_out.data_ptr(), k_pool.data_ptr(),
          v_pool.data_ptr(), cos.data_ptr(), sin.data_ptr(), positions.data_ptr(), seq_of_token.data_ptr(),
          block_table.data_ptr(), block_table.shape[1], num_heads, num_kv_heads, head_dim, page_size, n_pages,
          int(kv_layout), _stream())


def attention_generic(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, out: torch.Tensor,
                      positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor, *,
                      num_heads: int, scale: float, softcap: Optional[float], window: Optional[int],
                      max_position: int, full_precision: bool, bias_slopes: Optional[torch.Tensor] = None,
                      gate: Optional[torch.Tensor] = None) -> None:
    """bias_slopes: float32 [num_heads]; head h's capped score of key k for the query at position p gets
    bias_slopes[h] * (k - p) added before the softmax.  The value pool's last size is the value head size
    (out: [T, heads * that]).  gate: [T, >= num_heads] in q's dtype, rows of any stride (a column slice of a
    wider tensor): head h's output is multiplied by sigmoid(gate[t, h])."""
    T = q.shape[0]
    dt = q.dtype
    if k_pool.dim() != 4 or v_pool.dim() != 4:
        raise HipLibraryError("k_pool must be [pages, nKV, page, d]")
    n_pages, nKV, page_size, d = k_pool.shape
    dv = v_pool.shape[3]
    _dev(q, "q", None, (T, num_heads * d))
    _dev(out, "out", dt, (T, num_heads * dv))
    _dev(k_pool, "k_pool", dt)
    _dev(v_pool, "v_pool", dt, tuple(k_pool.shape[:3]) + (dv,))
    gate_ptr, gate_stride = None, 0
    if gate is not None:
        if (not gate.is_cuda or gate.dtype != dt or gate.dim() != 2 or gate.shape[0] != T or gate.shape[1] < num_heads
                or gate.stride(1) != 1 or gate.stride(0) < num_heads):
            raise HipLibraryError(f"gate must be [{T}, >= {num_heads}] {dt} with unit column stride")
        gate_ptr, gate_stride = gate.data_ptr(), gate.stride(0)
    _dev(positions, "positions", torch.int32, (T,))
    _dev(seq_of_token, "seq_of_token", torch.int32, (T,))
    _dev(block_table, "block_table", torch.int32)
    if block_table.dim() != 2 or max_position // page_size >= block_table.shape[1]:
        raise HipLibraryError(f"position {max_position} is beyond the block table {tuple(block_table.shape)}")
    if bias_slopes is not None:
        _dev(bias_slopes, "bias_slopes", torch.float32, (num_heads,))
    _call("alice_attention_generic", q.data_ptr(), dtype_code(dt), k_pool.data_ptr(), v_pool.data_ptr(),
          out.data_ptr(), positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
          block_table.shape[1], T, num_heads, nKV, d, page_size, float(scale),
          float(softcap or 0.0), int(window or 0), None if bias_slopes is None else bias_slopes.data_ptr(),
          int(full_precision), int(dv), gate_ptr, int(gate_stride), _stream())


def attention_masked(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, out: Optional[torch.Tensor],
                     positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor, *,
                     num_heads: int, scale: float, max_position: int, full_precision: bool,
                     softcap: Optional[float] = None, window: Optional[int] = None, chunk: Optional[int] = None,
                     keep_first: int = 0, bias_slopes: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None,
                     gate: Optional[torch.Tensor] = None, gate_per_element: bool = False, out_scale: float = 1.0,
                     value_cos: Optional[torch.Tensor] = None, value_sin: Optional[torch.Tensor] = None,
                     per_value_head: Optional[torch.Tensor] = None) -> None:
    """attention_generic with further masks and softmax terms over a row-major cache.  chunk: a query sees the keys
    of its own chunk of that many positions (counted from position 0); keep_first: keys below that position stay
    visible beside the window; sink: float32 [heads], a term of the denominator without a value; gate: float32
    [T, >= heads] (rows of any stride), with gate_per_element [T, >= heads * dv], one number an output element;
    out_scale: a constant factor of the gated output; value_cos / value_sin: float32
    [positions, dv / 2], the output of a head is turned back by the query's position (the values were cached turned
    by their own); per_value_head: float32 [T, heads, kv heads, dv] that receives every head's weights applied to
    each kv head's values (nothing goes to out, and no gate is applied: mix_heads follows)."""
    T = q.shape[0]
    dt = q.dtype
    if k_pool.dim() != 4 or v_pool.dim() != 4:
        raise HipLibraryError("k_pool must be [pages, nKV, page, d]")
    n_pages, nKV, page_size, d = k_pool.shape
    dv = v_pool.shape[3]
    _dev(q, "q", None, (T, num_heads * d))
    _dev(k_pool, "k_pool", dt)
    _dev(v_pool, "v_pool", dt, tuple(k_pool.shape[:3]) + (dv,))
    if per_value_head is not None:
        _dev(per_value_head, "per_value_head", torch.float32, (T, num_heads, nKV, dv))
        if gate is not None:
            raise HipLibraryError("per-value-head outputs take no gate: the mix that follows does")
    else:
        _dev(out, "out", dt, (T, num_heads * dv))
    gate_ptr, gate_stride = None, 0
    if gate is not None:
        need = num_heads * dv if gate_per_element else num_heads
        if (not gate.is_cuda or gate.dtype != torch.float32 or gate.dim() != 2 or gate.shape[0] != T or gate.shape[1] < need
                or gate.stride(1) != 1 or gate.stride(0) < need):
            raise HipLibraryError(f"gate must be [{T}, >= {need}] float32 with unit column stride")
        gate_ptr, gate_stride = gate.data_ptr(), gate.stride(0)
    _dev(positions, "positions", torch.int32, (T,))
    _dev(seq_of_token, "seq_of_token", torch.int32, (T,))
    _dev(block_table, "block_table", torch.int32)
    if block_table.dim() != 2 or max_position // page_size >= block_table.shape[1]:
        raise HipLibraryError(f"position {max_position} is beyond the block table {tuple(block_table.shape)}")
    if bias_slopes is not None:
        _dev(bias_slopes, "bias_slopes", torch.float32, (num_heads,))
    if sink is not None:
        _dev(sink, "sink", torch.float32, (num_heads,))
    if value_cos is not None:
        if dv % 2 or value_cos.dim() != 2 or value_cos.shape[1] != dv // 2 or value_sin.shape != value_cos.shape:
            raise HipLibraryError(f"value tables must be [positions, {dv // 2}]")
        _dev(value_cos, "value_cos", torch.float32)
        _dev(value_sin, "value_sin", torch.float32)
        if max_position >= value_cos.shape[0]:
            raise HipLibraryError(f"position {max_position} is beyond the rotation tables ({value_cos.shape[0]} positions)")
    _call("alice_attention_masked", q.data_ptr(), dtype_code(dt), k_pool.data_ptr(), v_pool.data_ptr(),
          None if out is None else out.data_ptr(), positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
          block_table.shape[1], T, num_heads, nKV, d, page_size, float(scale), float(softcap or 0.0), int(window or 0),
          None if bias_slopes is None else bias_slopes.data_ptr(), int(full_precision), int(dv), gate_ptr, int(gate_stride),
          2 if gate_per_element else 1, float(out_scale), int(chunk or 0), int(keep_first or 0), None if sink is None else sink.data_ptr(),
          None if value_cos is None else value_cos.data_ptr(), None if value_sin is None else value_sin.data_ptr(),
          None if per_value_head is None else per_value_head.data_ptr(), _stream())


def attention_tiled_supported(dtype: torch.dtype, head_dim: int, value_head_dim: int) -> bool:
    """Whether attention_tiled takes these operands: bfloat16 and head sizes that are multiples of 8 up to 256."""
    return dtype == torch.bfloat16 and bool(library().alice_attention_tiled_supported(int(head_dim), int(value_head_dim)))


def attention_tiled(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, out: Optional[torch.Tensor], ctx,
                    block_table: torch.Tensor, *, num_heads: int, scale: float, window: Optional[int] = None,
                    chunk: Optional[int] = None, keep_first: int = 0, bias_slopes: Optional[torch.Tensor] = None,
                    sink: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None, gate_per_element: bool = False,
                    out_scale: float = 1.0, value_cos: Optional[torch.Tensor] = None, value_sin: Optional[torch.Tensor] = None,
                    per_value_head: Optional[torch.Tensor] = None, heads_per_wave: int = 0) -> None:
    """attention_masked's result for bfloat16 prompts by the matrix-core kernel over the row-major cache (see
    attention_tiled.hip): `ctx` gives positions, cu_seqlens and the step's sizes; every sequence's tokens stand at
    consecutive positions.  heads_per_wave: how many heads of a kv head's group a wave takes (0: the launcher's
    choice by the step's size; 1, 2 or 4).  The other arguments are attention_masked's."""
    T = q.shape[0]
    if k_pool.dim() != 4 or v_pool.dim() != 4:
        raise HipLibraryError("k_pool must be [pages, nKV, page, d]")
    n_pages, nKV, page_size, d = k_pool.shape
    dv = v_pool.shape[3]
    _dev(q, "q", torch.bfloat16, (T, num_heads * d))
    _dev(k_pool, "k_pool", torch.bfloat16)
    _dev(v_pool, "v_pool", torch.bfloat16, tuple(k_pool.shape[:3]) + (dv,))
    if per_value_head is not None:
        _dev(per_value_head, "per_value_head", torch.float32, (T, num_heads, nKV, dv))
        if gate is not None:
            raise HipLibraryError("per-value-head outputs take no gate: the mix that follows does")
    else:
        _dev(out, "out", torch.bfloat16, (T, num_heads * dv))
    gate_ptr, gate_stride = None, 0
    if gate is not None:
        need = num_heads * dv if gate_per_element else num_heads
        if (not gate.is_cuda or gate.dtype != torch.float32 or gate.dim() != 2 or gate.shape[0] != T or gate.shape[1] < need
                or gate.stride(1) != 1 or gate.stride(0) < need):
            raise HipLibraryError(f"gate must be [{T}, >= {need}] float32 with unit column stride")
        gate_ptr, gate_stride = gate.data_ptr(), gate.stride(0)
    _dev(ctx.positions, "positions", torch.int32)
    _dev(ctx.cu_seqlens, "cu_seqlens", torch.int32)
    _dev(block_table, "block_table", torch.int32)
    if ctx.positions.numel() < T or ctx.cu_seqlens.numel() < ctx.n_seqs + 1:
        raise HipLibraryError("positions and cu_seqlens are too short for the step")
    if block_table.dim() != 2 or block_table.shape[0] < ctx.n_seqs or ctx.max_position // page_size >= block_table.shape[1]:
        raise HipLibraryError(f"position {ctx.max_position} is beyond the block table {tuple(block_table.shape)}")
    if bias_slopes is not None:
        _dev(bias_slopes, "bias_slopes", torch.float32, (num_heads,))
    if sink is not None:
        _dev(sink, "sink", torch.float32, (num_heads,))
    if value_cos is not None:
        if dv % 2 or value_cos.dim() != 2 or value_cos.shape[1] != dv // 2 or value_sin.shape != value_cos.shape:
            raise HipLibraryError(f"value tables must be [positions, {dv // 2}]")
        _dev(value_cos, "value_cos", torch.float32)
        _dev(value_sin, "value_sin", torch.float32)
        if ctx.max_position >= value_cos.shape[0]:
            raise HipLibraryError(f"position {ctx.max_position} is beyond the rotation tables ({value_cos.shape[0]} positions)")
    _call("alice_attention_tiled", q.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), None if out is None else out.data_ptr(),
          None if per_value_head is None else per_value_head.data_ptr(), ctx.positions.data_ptr(), ctx.cu_seqlens.data_ptr(),
          block_table.data_ptr(), block_table.shape[1], T, int(ctx.n_seqs), num_heads, nKV, d, dv, page_size, float(scale),
          int(window or 0), int(chunk or 0), int(keep_first or 0), None if bias_slopes is None else bias_slopes.data_ptr(),
          None if sink is None else sink.data_ptr(), None if value_cos is None else value_cos.data_ptr(),
          None if value_sin is None else value_sin.data_ptr(), gate_ptr, int(gate_stride), 2 if gate_per_element else 1,
          float(out_scale), int(heads_per_wave), _stream())


def attention_split_supported(dtype: torch.dtype, num_heads: int, num_kv_heads: int, head_dim: int, value_head_dim: int) -> bool:
    """Whether attention_split takes these operands: groups of at most 16 query heads a kv head, head sizes that are
    multiples of 16 bytes up to 256."""
    return bool(library().alice_attention_split_supported(dtype_code(dtype), int(num_heads), int(num_kv_heads), int(head_dim),
                                                          int(value_head_dim)))


def attention_split(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, out: Optional[torch.Tensor],
                    positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor, *, num_heads: int,
                    scale: float, max_position: int, max_keys: int, window: Optional[int] = None, chunk: Optional[int] = None,
                    keep_first: int = 0, bias_slopes: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None,
                    gate: Optional[torch.Tensor] = None, gate_per_element: bool = False, out_scale: float = 1.0,
                    value_cos: Optional[torch.Tensor] = None, value_sin: Optional[torch.Tensor] = None,
                    per_value_head: Optional[torch.Tensor] = None) -> None:
    """attention_masked's result with the keys split over blocks (see attention_split.hip): the kernel of steps of
    single tokens, in either dtype.  max_keys: the most keys any token of the step sees (from the step's longest
    context and the mask); the other arguments are attention_masked's."""
    T = q.shape[0]
    dt = q.dtype
    if k_pool.dim() != 4 or v_pool.dim() != 4:
        raise HipLibraryError("k_pool must be [pages, nKV, page, d]")
    n_pages, nKV, page_size, d = k_pool.shape
    dv = v_pool.shape[3]
    _dev(q, "q", None, (T, num_heads * d))
    _dev(k_pool, "k_pool", dt)
    _dev(v_pool, "v_pool", dt, tuple(k_pool.shape[:3]) + (dv,))
    if per_value_head is not None:
        _dev(per_value_head, "per_value_head", torch.float32, (T, num_heads, nKV, dv))
        if gate is not None:
            raise HipLibraryError("per-value-head outputs take no gate: the mix that follows does")
    else:
        _dev(out, "out", dt, (T, num_heads * dv))
    gate_ptr, gate_stride = None, 0
    if gate is not None:
        need = num_heads * dv if gate_per_element else num_heads
        if (not gate.is_cuda or gate.dtype != torch.float32 or gate.dim() != 2 or gate.shape[0] != T or gate.shape[1] < need
                or gate.stride(1) != 1 or gate.stride(0) < need):
            raise HipLibraryError(f"gate must be [{T}, >= {need}] float32 with unit column stride")
        gate_ptr, gate_stride = gate.data_ptr(), gate.stride(0)
    _dev(positions, "positions", torch.int32, (T,))
    _dev(seq_of_token, "seq_of_token", torch.int32, (T,))
    _dev(block_table, "block_table", torch.int32)
    if block_table.dim() != 2 or max_position // page_size >= block_table.shape[1]:
        raise HipLibraryError(f"position {max_position} is beyond the block table {tuple(block_table.shape)}")
    if bias_slopes is not None:
        _dev(bias_slopes, "bias_slopes", torch.float32, (num_heads,))
    if sink is not None:
        _dev(sink, "sink", torch.float32, (num_heads,))
    if value_cos is not None:
        if dv % 2 or value_cos.dim() != 2 or value_cos.shape[1] != dv // 2 or value_sin.shape != value_cos.shape:
            raise HipLibraryError(f"value tables must be [positions, {dv // 2}]")
        _dev(value_cos, "value_cos", torch.float32)
        _dev(value_sin, "value_sin", torch.float32)
        if max_position >= value_cos.shape[0]:
            raise HipLibraryError(f"position {max_position} is beyond the rotation tables ({value_cos.shape[0]} positions)")
    if max_keys < 1 or max_keys > max_position + 1:
        max_keys = max_position + 1
    lib = library()
    runs = lib.alice_attention_split_runs(int(max_keys))
    work = torch.empty((lib.alice_attention_split_workspace(T, num_heads, nKV, dv, runs, int(per_value_head is not None)),),
                       dtype=torch.float32, device=q.device)
    _call("alice_attention_split", q.data_ptr(), dtype_code(dt), k_pool.data_ptr(), v_pool.data_ptr(),
          None if out is None else out.data_ptr(), None if per_value_head is None else per_value_head.data_ptr(),
          positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(), block_table.shape[1], T, num_heads, nKV, d, dv,
          page_size, float(scale), int(window or 0), int(chunk or 0), int(keep_first or 0), int(max_keys),
          None if bias_slopes is None else bias_slopes.data_ptr(), None if sink is None else sink.data_ptr(),
          None if value_cos is None else value_cos.data_ptr(), None if value_sin is None else value_sin.data_ptr(),
          gate_ptr, int(gate_stride), 2 if gate_per_element else 1, float(out_scale), work.data_ptr(), _stream())


def mix_heads(a: torch.Tensor, talk: torch.Tensor, gate: Optional[torch.Tensor], out: torch.Tensor, *,
              full_precision: bool, out_scale: float = 1.0) -> None:
    """out[t, h, :] = out_scale * sigmoid(gate[t, h, :]) * sum_g talk[h, g] * a[t, g, kv head of h, :]; a: float32
    [T, heads, kv heads, dv]; talk: float32 [heads, heads]; gate: float32 [T, >= heads * dv] (or None)."""
    if a.dim() != 4:
        raise HipLibraryError("a must be [T, heads, kv heads, dv]")
    T, H, G, dv = a.shape
    _dev(a, "a", torch.float32)
    _dev(talk, "talk", torch.float32, (H, H))
    _dev(out, "out", None, (T, H * dv))
    gate_ptr, gate_stride = None, 0
    if gate is not None:
        if (not gate.is_cuda or gate.dtype != torch.float32 or gate.dim() != 2 or gate.shape[0] != T or gate.shape[1] < H * dv
                or gate.stride(1) != 1):
            raise HipLibraryError(f"gate must be [{T}, >= {H * dv}] float32 with unit column stride")
        gate_ptr, gate_stride = gate.data_ptr(), gate.stride(0)
    _call("alice_mix_heads", a.data_ptr(), talk.data_ptr(), gate_ptr, int(gate_stride), float(out_scale), out.data_ptr(),
          dtype_code(out.dtype), T, H, G, dv, int(full_precision), _stream())


def qkv_prepare(rows: torch.Tensor, bias: Optional[torch.Tensor], q_out: torch.Tensor, k_pool: Optional[torch.Tensor],
                v_pool: Optional[torch.Tensor], positions: torch.Tensor, seq_of_token: Optional[torch.Tensor],
                block_table: Optional[torch.Tensor], *, num_heads: int, num_kv_heads: int, head_dim: int,
                value_head_dim: int, max_position: int, cos: Optional[torch.Tensor] = None,
                sin: Optional[torch.Tensor] = None, rotary_dim: int = 0, interleaved: bool = True,
                value_cos: Optional[torch.Tensor] = None, value_sin: Optional[torch.Tensor] = None,
                norm_weight: Optional[torch.Tensor] = None, norm_eps: float = 0.0) -> None:
    """From the rows [q | k | v | ...] of a fused projection (float32, or q_out's dtype): bias [>= q, k, v columns]
    added, q and k heads rotated over their first rotary_dim dimensions in pairs ((2i, 2i + 1) if interleaved, else
    (i, i + rotary_dim / 2)) from tables [positions, rotary_dim / 2], values turned over all their dimensions where
    value tables [positions, dv / 2] are given; q to q_out, k and v into the row-major pools at their positions.
    norm_weight: float32 [q columns + k columns (where a cache is written)]: after the bias and before the rotation, the q
    columns (all heads together) and the k columns are each divided by their root mean square over the whole projection
    (norm_eps inside the root) and multiplied by this weight."""
    T = rows.shape[0]
    dt = q_out.dtype
    d, dv = head_dim, value_head_dim
    if rows.dim() != 2 or rows.dtype not in (torch.float32, dt):
        raise HipLibraryError("rows must be [T, width] in float32 or the outputs' dtype")
    _dev(rows, "rows")
    width = num_heads * d + (num_kv_heads * (d + dv) if k_pool is not None else 0)
    if rows.shape[1] < width:
        raise HipLibraryError(f"rows of {tuple(rows.shape)} are too short for the heads")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() < width:
            raise HipLibraryError(f"bias must hold {width} elements")
    _dev(q_out, "q_out", None, (T, num_heads * d))
    _dev(positions, "positions", torch.int32, (T,))
    for c, s_, n, what in ((cos, sin, rotary_dim, "cos/sin"), (value_cos, value_sin, dv, "value tables")):
        if c is not None:
            if c.dim() != 2 or c.shape[1] != n // 2 or s_.shape != c.shape or n % 2:
                raise HipLibraryError(f"{what} must be [positions, {n // 2}]")
            _dev(c, what, torch.float32)
            _dev(s_, what, torch.float32)
            if max_position >= c.shape[0]:
                raise HipLibraryError(f"position {max_position} is beyond the rotation tables ({c.shape[0]} positions)")
    page_size = n_pages = bt_stride = 0
    if k_pool is not None:
        if k_pool.dim() != 4 or k_pool.shape[1] != num_kv_heads or k_pool.shape[3] != d:
            raise HipLibraryError(f"k_pool must be [pages, {num_kv_heads}, page, {d}], found {tuple(k_pool.shape)}")
        _dev(k_pool, "k_pool", dt)
        _dev(v_pool, "v_pool", dt, tuple(k_pool.shape[:3]) + (dv,))
        n_pages, _, page_size, _ = k_pool.shape
        _dev(seq_of_token, "seq_of_token", torch.int32, (T,))
        _dev(block_table, "block_table", torch.int32)
        if block_table.dim() != 2 or max_position // page_size >= block_table.shape[1]:
            raise HipLibraryError(f"position {max_position} is beyond the block table")
        bt_stride = block_table.shape[1]
    inv_rms = None
    if norm_weight is not None:
        n_norm = num_heads * d + (num_kv_heads * d if k_pool is not None else 0)
        _dev(norm_weight, "norm_weight", torch.float32, (n_norm,))
        if not norm_eps > 0:
            raise HipLibraryError("the projection norm needs a positive eps")
        inv_rms = torch.empty((T, 2), dtype=torch.float32, device=rows.device)
    _call("alice_qkv_prepare", rows.data_ptr(), dtype_code(rows.dtype), rows.shape[1], _opt(bias, "bias"), q_out.data_ptr(),
          _opt(k_pool, "k_pool"), _opt(v_pool, "v_pool"), dtype_code(dt), _opt(cos, "cos"), _opt(sin, "sin"),
          int(rotary_dim if cos is not None else 0), int(interleaved), _opt(value_cos, "value_cos"), _opt(value_sin, "value_sin"),
          positions.data_ptr(), _opt(seq_of_token, "seq_of_token"), _opt(block_table, "block_table"), bt_stride, T,
          num_heads, num_kv_heads if k_pool is not None else 0, d, dv, page_size, n_pages,
          _opt(norm_weight, "norm_weight"), float(norm_eps), _opt(inv_rms, "inv_rms"), _stream())


def add_rows(x: torch.Tensor, rows: Optional[torch.Tensor], vector: Optional[torch.Tensor]) -> None:
    """x[t, :] += rows[t, :] + vector (either may be None); all float32."""
    T, W = x.shape
    _dev(x, "x", torch.float32)
    _call("alice_add_rows", x.data_ptr(), _opt(rows, "rows", torch.float32, (T, W)), _opt(vector, "vector", torch.float32, (W,)),
          T, W, _stream())



# ------------------------------------------------------------------------------------ latent attention

LATENT_MAX_RANK = 1024       # the largest latent the latent attention kernels take


def _latent_pool(k_pool: torch.Tensor, kv_rank: int, rot_dim: int, dt) -> None:
    if k_pool.dim() != 4 or k_pool.shape[1] != 1 or k_pool.shape[3] != kv_rank + rot_dim:
        raise HipLibraryError(f"k_pool must be [pages, 1, page, {kv_rank + rot_dim}], found {tuple(k_pool.shape)}")
    _dev(k_pool, "k_pool", dt)


def _rot_tables(cos, sin, rot_dim: int, max_position: int):
    if rot_dim == 0:
        return None, None
    if cos is None or sin is None or cos.dim() != 2 or cos.shape[1] != rot_dim // 2 or sin.shape != cos.shape or rot_dim % 2:
        raise HipLibraryError(f"cos/sin must be [positions, {rot_dim // 2}]")
    if max_position >= cos.shape[0]:
        raise HipLibraryError(f"position {max_position} is beyond the rotation tables ({cos.shape[0]} positions)")
    return _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32)


def latent_prepare(rows: torch.Tensor, w_q: torch.Tensor, w_kv: torch.Tensor, q_latent: torch.Tensor,
                   k_pool: Optional[torch.Tensor], positions: torch.Tensor, seq_of_token: Optional[torch.Tensor],
                   block_table: Optional[torch.Tensor], *, q_rank: int, kv_rank: int, rot_dim: int, eps: float,
                   cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], max_position: int) -> None:
    """From the float32 rows [a (q_rank) | c (kv_rank) | kr (rot_dim)] of a fused down projection: the RMS-normed a
    (weight w_q) to q_latent [T, q_rank]; the RMS-normed c (weight w_kv) and kr rotated in pairs (2i, 2i + 1) into the
    token's row of the cache, [pages, 1, page, kv_rank + rot_dim] (None: nothing is cached)."""
    T = rows.shape[0]
    if rows.dim() != 2 or rows.shape[1] < q_rank + kv_rank + rot_dim:
        raise HipLibraryError(f"rows must be [T, >= {q_rank + kv_rank + rot_dim}], found {tuple(rows.shape)}")
    _dev(rows, "rows", torch.float32)
    _dev(w_q, "w_q", torch.float32, (q_rank,))
    _dev(w_kv, "w_kv", torch.float32, (kv_rank,))
    _dev(q_latent, "q_latent", None, (T, q_rank))
    _dev(positions, "positions", torch.int32, (T,))
    c, s_ = _rot_tables(cos, sin, rot_dim, max_position)
    page_size = n_pages = bt_stride = 0
    if k_pool is not None:
        _latent_pool(k_pool, kv_rank, rot_dim, q_latent.dtype)
        n_pages, _, page_size, _ = k_pool.shape
        _dev(seq_of_token, "seq_of_token", torch.int32, (T,))
        _dev(block_table, "block_table", torch.int32)
        if block_table.dim() != 2 or max_position // page_size >= block_table.shape[1]:
            raise HipLibraryError(f"position {max_position} is beyond the block table")
        bt_stride = block_table.shape[1]
    _call("alice_latent_prepare", rows.data_ptr(), rows.shape[1], q_rank, kv_rank, rot_dim, w_q.data_ptr(), w_kv.data_ptr(),
          float(eps), c, s_, positions.data_ptr(), _opt(seq_of_token, "seq_of_token"), _opt(block_table, "block_table"),
          bt_stride, page_size, n_pages, q_latent.data_ptr(), _opt(k_pool, "k_pool"), dtype_code(q_latent.dtype), T, _stream())


def heads_linear(x: torch.Tensor, wt: torch.Tensor, y: torch.Tensor, *, heads: int, n: int, k: int, rot_dim: int = 0,
                 cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None,
                 positions: Optional[torch.Tensor] = None, max_position: int = 0) -> None:
    """A matrix a head: y[t, h, 0:n] = M_h x[t, h, 0:k] with M given transposed, wt [heads, k, n]; x [T, heads * (k +
    rot_dim)], y [T, heads * (n + rot_dim)]; the rot_dim elements behind a head's k inputs are rotated in pairs
    (2i, 2i + 1) by the token's position and put behind its n outputs."""
    T = x.shape[0]
    _dev(x, "x", None, (T, heads * (k + rot_dim)))
    _dev(y, "y", None, (T, heads * (n + rot_dim)))
    _dev(wt, "wt", None, (heads, k, n))
    c, s_ = _rot_tables(cos, sin, rot_dim, max_position)
    if rot_dim:
        _dev(positions, "positions", torch.int32, (T,))
    _call("alice_heads_linear", x.data_ptr(), dtype_code(x.dtype), heads * (k + rot_dim), k + rot_dim, wt.data_ptr(),
          dtype_code(wt.dtype), y.data_ptr(), dtype_code(y.dtype), heads * (n + rot_dim), n + rot_dim, T, heads, n, k,
          rot_dim, c, s_, positions.data_ptr() if rot_dim else None, _stream())


def heads_linear_mfma_supported(dtype: torch.dtype, n: int, k: int, rot_dim: int = 0) -> bool:
    return dtype == torch.bfloat16 and bool(library().alice_heads_linear_mfma_supported(int(n), int(k), int(rot_dim)))


def heads_linear_mfma(x: torch.Tensor, w: torch.Tensor, y: torch.Tensor, *, heads: int, n: int, k: int, rot_dim: int = 0,
                      cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None,
                      positions: Optional[torch.Tensor] = None, max_position: int = 0) -> None:
    """heads_linear on the matrix cores: bfloat16 throughout, and the matrices as stored, w [heads, n, k]."""
    T = x.shape[0]
    _dev(x, "x", torch.bfloat16, (T, heads * (k + rot_dim)))
    _dev(y, "y", torch.bfloat16, (T, heads * (n + rot_dim)))
    _dev(w, "w", torch.bfloat16, (heads, n, k))
    c, s_ = _rot_tables(cos, sin, rot_dim, max_position)
    if rot_dim:
        _dev(positions, "positions", torch.int32, (T,))
    _call("alice_heads_linear_mfma", x.data_ptr(), heads * (k + rot_dim), k + rot_dim, w.data_ptr(), y.data_ptr(),
          heads * (n + rot_dim), n + rot_dim, T, heads, n, k, rot_dim, c, s_, positions.data_ptr() if rot_dim else None,
          _stream())


def latent_attention(q: torch.Tensor, k_pool: torch.Tensor, out: torch.Tensor, ctx, block_table: torch.Tensor, *,
                     num_heads: int, kv_rank: int, rot_dim: int, scale: float, window: Optional[int],
                     full_precision: bool) -> None:
    """Softmax attention of q [T, heads * (kv_rank + rot_dim)] over the cached rows [latent | rotated part] of each
    token's sequence, keys max(0, pos + 1 - window) .. pos; out [T, heads * kv_rank] = the weights times the rows'
    latents.  32-bit arithmetic, any sizes up to LATENT_MAX_RANK."""
    T = q.shape[0]
    dt = q.dtype
    _latent_pool(k_pool, kv_rank, rot_dim, dt)
    if not 1 <= kv_rank <= LATENT_MAX_RANK:
        raise HipLibraryError(f"latent size {kv_rank} is outside 1..{LATENT_MAX_RANK}")
    _dev(q, "q", None, (T, num_heads * (kv_rank + rot_dim)))
    _dev(out, "out", dt, (T, num_heads * kv_rank))
    _dev(ctx.positions, "positions", torch.int32, (T,))
    _dev(ctx.seq_of_token, "seq_of_token", torch.int32, (T,))
    _dev(block_table, "block_table", torch.int32)
    page_size = k_pool.shape[2]
    if block_table.dim() != 2 or ctx.max_position // page_size >= block_table.shape[1] or block_table.shape[0] < ctx.n_seqs:
        raise HipLibraryError(f"position {ctx.max_position} is beyond the block table")
    _call("alice_latent_attention", q.data_ptr(), dtype_code(dt), k_pool.data_ptr(), out.data_ptr(), ctx.positions.data_ptr(),
          ctx.seq_of_token.data_ptr(), block_table.data_ptr(), block_table.shape[1], T, num_heads, kv_rank, rot_dim, page_size,
          float(scale), int(window or 0), int(full_precision), _stream())


def latent_tiled_supported(dtype: torch.dtype, kv_rank: int, rot_dim: int) -> bool:
    return dtype == torch.bfloat16 and bool(library().alice_latent_tiled_supported(int(kv_rank), int(rot_dim)))


def latent_tiled_splits(n_tokens: int, num_heads: int, max_keys: int) -> int:
    """Over how many blocks a row group's keys are spread in a step of single tokens: enough for two blocks a CU (a
    token's heads are a group of their own, 64 rows at most; measured fastest at 1, 8 and 64 tokens of 16 heads over
    1,024 and 8,192 keys), every block with at least two runs of 32 keys."""
    groups = n_tokens * -(-num_heads // 64)
    key_blocks = -(-max(1, max_keys) // 32) + 1
    most = min(library().alice_latent_tiled_max_splits(), key_blocks // 2)
    return max(1, min(most, 512 // max(1, groups)))


def latent_attention_tiled(q: torch.Tensor, k_pool: torch.Tensor, out: torch.Tensor, ctx, block_table: torch.Tensor, *,
                           num_heads: int, kv_rank: int, rot_dim: int, scale: float, window: Optional[int],
                           splits: int = 1, single_tokens: bool = False) -> None:
    """latent_attention on the matrix cores (bfloat16; sizes as latent_tiled_supported says).  The step's tokens are
    those of ctx.n_seqs sequences in order (ctx.cu_seqlens), each at consecutive positions.  splits > 1 spreads every
    group of 64 query rows (token, head) over that many blocks along the keys.  single_tokens: every sequence of the
    step brings exactly one token (a decode step); with at most 16 heads the kernel of such steps then runs."""
    T = q.shape[0]
    _latent_pool(k_pool, kv_rank, rot_dim, torch.bfloat16)
    _dev(q, "q", torch.bfloat16, (T, num_heads * (kv_rank + rot_dim)))
    _dev(out, "out", torch.bfloat16, (T, num_heads * kv_rank))
    _dev(ctx.positions, "positions", torch.int32, (T,))
    _dev(ctx.cu_seqlens, "cu_seqlens", torch.int32)
    _dev(block_table, "block_table", torch.int32)
    page_size = k_pool.shape[2]
    if ctx.cu_seqlens.numel() < ctx.n_seqs + 1:
        raise HipLibraryError("cu_seqlens is shorter than the step's sequences")
    if single_tokens and T != ctx.n_seqs:
        raise HipLibraryError(f"a step of single tokens has {T} tokens for {ctx.n_seqs} sequences")
    if block_table.dim() != 2 or ctx.max_position // page_size >= block_table.shape[1] or block_table.shape[0] < ctx.n_seqs:
        raise HipLibraryError(f"position {ctx.max_position} is beyond the block table")
    part = None
    if splits > 1:
        part = torch.empty((splits * T * num_heads * (kv_rank + 2),), dtype=torch.float32, device=q.device)
    _call("alice_latent_tiled", q.data_ptr(), k_pool.data_ptr(), out.data_ptr(), _opt(part, "part"), ctx.positions.data_ptr(),
          ctx.cu_seqlens.data_ptr(), block_table.data_ptr(), block_table.shape[1], T, ctx.n_seqs, num_heads, kv_rank, rot_dim,
          page_size, float(scale), int(window or 0), int(splits), int(bool(single_tokens)), _stream())


GLA_MAX_KEY_DIM = 256       # the largest key size the gated linear attention kernel keeps in registers


def gla(rows: torch.Tensor, z: torch.Tensor, z_bias: torch.Tensor, norm_w: torch.Tensor, out: torch.Tensor, ctx,
        S: torch.Tensor, *, heads: int, head_dim: int, value_head_dim: int, tau: float, q_scale: float, eps: float,
        columns, out_scale: float = 1.0, columns_per_block: int = 0) -> None:
    """Gated linear attention over a step (`ctx` gives cu_seqlens, slots, n_seqs): rows float32 [T, width] with q, k,
    v and the gate at `columns` = (q, k, v, g); z float32 [T, heads * d] and z_bias float32 [heads * d]: the decay is
    sigmoid(z + z_bias)^(1 / tau), which is left in z; S float32 [slots, heads, d, dv]; out [T, heads * dv], times out_scale.  columns_per_block: 0 lets the launcher
    choose by the step's size; 8, 16 or 64 fix the value columns a block."""
    H, d, dv = heads, head_dim, value_head_dim
    T = rows.shape[0]
    _dev(rows, "rows", torch.float32)
    _dev(z, "z", torch.float32, (T, H * d))
    _dev(z_bias, "z_bias", torch.float32, (H * d,))
    _dev(norm_w, "norm_w", None, (dv,))
    _dev(out, "out", None, (T, H * dv))
    _dev(ctx.cu_seqlens, "cu_seqlens", torch.int32)
    _dev(ctx.slots, "slots", torch.int32)
    if ctx.cu_seqlens.numel() < ctx.n_seqs + 1 or ctx.slots.numel() < ctx.n_seqs:
        raise HipLibraryError("cu_seqlens and slots are too short for the step's sequences")
    n_slots = S.shape[0]
    _dev(S, "S", torch.float32, (n_slots, H, d, dv))
    work = torch.empty((T, H * dv), dtype=torch.float32, device=rows.device)
    q_col, k_col, v_col, g_col = (int(c) for c in columns)
    _call("alice_gla", rows.data_ptr(), rows.shape[1], q_col, k_col, v_col, g_col, z.data_ptr(), z_bias.data_ptr(), float(tau),
          float(q_scale), float(out_scale), norm_w.data_ptr(), dtype_code(norm_w.dtype), float(eps), out.data_ptr(), dtype_code(out.dtype),
          _opt(work, "work"), ctx.cu_seqlens.data_ptr(), ctx.slots.data_ptr(), S.data_ptr(), T, int(ctx.n_seqs), int(n_slots),
          H, d, dv, int(columns_per_block), _stream())


# ------------------------------------------------------------------------------------ recurrent mixers

SHORT_CONV_MAX_TAPS = 16        # the most taps the short convolution takes
RECURRENCE_MAX_KEY_DIM = 256    # the largest key size the matrix recurrence keeps in registers
ROUTER_MAX_EXPERTS = 1024       # the most experts the router's kernel ranks


def _step_arrays(ctx) -> None:
    _dev(ctx.cu_seqlens, "cu_seqlens", torch.int32)
    _dev(ctx.slots, "slots", torch.int32)
    if ctx.cu_seqlens.numel() < ctx.n_seqs + 1 or ctx.slots.numel() < ctx.n_seqs:
        raise HipLibraryError("cu_seqlens and slots are too short for the step's sequences")


def short_conv(rows: torch.Tensor, col0: int, weight: torch.Tensor, bias: Optional[torch.Tensor], state: Optional[torch.Tensor],
               out: torch.Tensor, ctx, *, silu: bool = True) -> None:
    """out[t, c] = act(bias[c] + sum_j weight[c, j] x[t - (taps - 1) + j, c]) with x = rows[:, col0 + c] (float32), over the
    tokens of the token's own sequence; what lies before the step comes from state float32 [slots, channels, taps - 1]
    (the last inputs of the sequence's earlier steps, zeros at its start), which then takes the step's last inputs."""
    T = rows.shape[0]
    if weight.dim() != 2:
        raise HipLibraryError("weight must be [channels, taps]")
    C, taps = weight.shape
    _dev(rows, "rows", torch.float32)
    if rows.dim() != 2 or col0 < 0 or col0 + C > rows.shape[1]:
        raise HipLibraryError(f"rows of {tuple(rows.shape)} are too short for {C} channels from column {col0}")
    _dev(weight, "weight", torch.float32)
    _opt(bias, "bias", torch.float32, (C,))
    _dev(out, "out", torch.float32, (T, C))
    _step_arrays(ctx)
    _dev(ctx.seq_of_token, "seq_of_token", torch.int32)
    if ctx.seq_of_token.numel() < T:
        raise HipLibraryError("seq_of_token is too short for the step")
    if taps > 1:
        if state is None or state.dim() != 3 or tuple(state.shape[1:]) != (C, taps - 1):
            raise HipLibraryError(f"state must be [slots, {C}, {taps - 1}]")
        _dev(state, "state", torch.float32)
    _call("alice_short_conv", rows.data_ptr(), rows.shape[1], int(col0), C, taps, weight.data_ptr(), _opt(bias, "bias"),
          None if taps == 1 else state.data_ptr(), out.data_ptr(), int(bool(silu)), ctx.cu_seqlens.data_ptr(),
          ctx.seq_of_token.data_ptr(), ctx.slots.data_ptr(), T, int(ctx.n_seqs), _stream())


def ssm_prepare(rows: torch.Tensor, dt_col: int, dt_bias: torch.Tensor, a_log: torch.Tensor, step: torch.Tensor,
                decay: torch.Tensor) -> None:
    """step = softplus(rows[:, dt_col + h] + dt_bias[h]); decay = exp(-exp(a_log[h]) * step); float32 [T, heads] each."""
    T, H = step.shape
    _dev(rows, "rows", torch.float32)
    _dev(dt_bias, "dt_bias", torch.float32, (H,))
    _dev(a_log, "a_log", torch.float32, (H,))
    _dev(step, "step", torch.float32)
    _dev(decay, "decay", torch.float32, (T, H))
    if rows.shape[0] != T or dt_col + H > rows.shape[1]:
        raise HipLibraryError("rows do not hold the step sizes")
    _call("alice_ssm_prepare", rows.data_ptr(), rows.shape[1], int(dt_col), dt_bias.data_ptr(), a_log.data_ptr(), step.data_ptr(),
          decay.data_ptr(), T, H, _stream())


def delta_prepare(qk: torch.Tensor, k_col: int, z: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, rows: torch.Tensor,
                  b_col: int, beta: torch.Tensor, *, qk_heads: int, heads: int, head_dim: int, unit_eps: float, q_scale: float) -> None:
    """In place: the q heads (columns 0 .. qk_heads * d of qk) and the k heads (from k_col) become unit vectors
    x / sqrt(sum x^2 + unit_eps), q also times q_scale; z [T, heads * d] becomes exp(-exp(a_log[h]) softplus(z + dt_bias));
    beta[t, h] = sigmoid(rows[t, b_col + h])."""
    T = qk.shape[0]
    G, H, d = qk_heads, heads, head_dim
    _dev(qk, "qk", torch.float32)
    _dev(z, "z", torch.float32, (T, H * d))
    _dev(dt_bias, "dt_bias", torch.float32, (H * d,))
    _dev(a_log, "a_log", torch.float32, (H,))
    _dev(rows, "rows", torch.float32)
    _dev(beta, "beta", torch.float32, (T, H))
    if rows.shape[0] != T or b_col + H > rows.shape[1] or k_col < G * d or k_col + G * d > qk.shape[1]:
        raise HipLibraryError("the rows are too short for the heads")
    _call("alice_delta_prepare", qk.data_ptr(), qk.shape[1], int(k_col), G, d, float(unit_eps), float(q_scale), z.data_ptr(),
          dt_bias.data_ptr(), a_log.data_ptr(), rows.data_ptr(), rows.shape[1], int(b_col), beta.data_ptr(), T, H, _stream())


def recurrence_columns(n_seqs: int, heads: int, head_dim: int, value_head_dim: int) -> int:
    """The value columns a wave that matrix_recurrence chooses for a step of this many sequences.  A caller whose steps
    are also replayed from graphs recorded for a rounded-up number of sequences asks with that number and passes the answer
    on, so that both kinds of step add in the same order."""
    return library().alice_matrix_recurrence_columns(int(n_seqs), int(heads), int(head_dim), int(value_head_dim))


def matrix_recurrence(q, q_col: int, k, k_col: int, v, v_col: int, decay: torch.Tensor, b: torch.Tensor, skip: Optional[torch.Tensor],
                      out: torch.Tensor, ctx, S: torch.Tensor, *, heads: int, qk_heads: int, head_dim: int, value_head_dim: int,
                      delta: bool, decay_per_channel: bool, columns_per_wave: int = 0) -> None:
    """The recurrence of a matrix state a head over a step (`ctx` gives cu_seqlens, slots, n_seqs), all float32:
    delta False: S = diag(a) S + k (b v)^T; True: S = diag(a) S, u = b (v - S^T k), S += k u^T; then o = S^T q (+ skip[h] v).
    q, k: rows with the heads' columns from q_col / k_col, shared by groups of heads / qk_heads heads; v: rows with
    heads * dv columns from v_col; decay: [T, heads * d] (decay_per_channel) or [T, heads]; b: [T, heads]; S: [slots, heads, d, dv]; out: [T, heads * dv].
    columns_per_wave: 0 lets the launcher choose by the step's size; 4, 8 or 16 fix the value columns a wave."""
    H, d, dv = heads, head_dim, value_head_dim
    T = out.shape[0]
    for t_, nm in ((q, "q"), (k, "k"), (v, "v")):
        _dev(t_, nm, torch.float32)
        if t_.dim() != 2 or t_.shape[0] != T:
            raise HipLibraryError(f"{nm} must be [T, width]")
    if q_col + qk_heads * d > q.shape[1] or k_col + qk_heads * d > k.shape[1] or v_col + H * dv > v.shape[1]:
        raise HipLibraryError("the rows are too short for the heads")
    per_row = bool(decay_per_channel)
    _dev(decay, "decay", torch.float32, (T, H * d) if per_row else (T, H))
    _dev(b, "b", torch.float32, (T, H))
    _opt(skip, "skip", torch.float32, (H,))
    _dev(out, "out", torch.float32, (T, H * dv))
    _step_arrays(ctx)
    n_slots = S.shape[0]
    _dev(S, "S", torch.float32, (n_slots, H, d, dv))
    _call("alice_matrix_recurrence", q.data_ptr(), q.shape[1], int(q_col), k.data_ptr(), k.shape[1], int(k_col), v.data_ptr(),
          v.shape[1], int(v_col), decay.data_ptr(), int(per_row), b.data_ptr(), _opt(skip, "skip"), out.data_ptr(),
          ctx.cu_seqlens.data_ptr(), ctx.slots.data_ptr(), S.data_ptr(), int(ctx.n_seqs), int(n_slots), H, int(qk_heads), d, dv,
          int(bool(delta)), int(columns_per_wave), _stream())


def norm_gate(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, *, parts: int, eps: float, weight_shared: bool,
              gate: Optional[torch.Tensor] = None, gate_col: int = 0, gate_act: Optional[str] = None) -> None:
    """Rows of x (float32 [T, width]) in `parts` equal parts, each divided by its root mean square (eps inside the root)
    and multiplied by weight (float32, of the row's length, or with weight_shared of a part's length, the same for every part).
    gate_act "silu": times silu(gate[:, gate_col + .]) before the norm; "sigmoid": times sigmoid(.) after it."""
    T, width = x.shape
    _dev(x, "x", torch.float32)
    _dev(out, "out", None, (T, width))
    if width % parts:
        raise HipLibraryError(f"{parts} parts must divide the width {width}")
    _dev(weight, "weight", torch.float32, (width // parts if weight_shared else width,))
    act = {None: 0, "silu": 1, "sigmoid": 2}[gate_act]
    if act:
        _dev(gate, "gate", torch.float32)
        if gate.dim() != 2 or gate.shape[0] != T or gate_col + width > gate.shape[1]:
            raise HipLibraryError("the gate rows are too short")
    _call("alice_norm_gate", x.data_ptr(), width, int(parts), _opt(gate, "gate") if act else None, gate.shape[1] if act else 0,
          int(gate_col), act, weight.data_ptr(), int(bool(weight_shared)), float(eps), out.data_ptr(),
          dtype_code(out.dtype), T, _stream())


def route_topk(logits: torch.Tensor, bias: Optional[torch.Tensor], weights: torch.Tensor, top: int) -> None:
    """weights[t] = softmax over the `top` largest of logits[t] + bias at their places, zero elsewhere; float32 [T, experts]."""
    T, E = logits.shape
    _dev(logits, "logits", torch.float32)
    _opt(bias, "bias", torch.float32, (E,))
    _dev(weights, "weights", torch.float32, (T, E))
    _call("alice_route_topk", logits.data_ptr(), _opt(bias, "bias"), weights.data_ptr(), T, E, int(top), _stream())


def scale_columns(x: torch.Tensor, weights: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, e * F + j] = x[t, e * F + j] * weights[t, e] for x [T, experts * F] and float32 weights [T, experts]."""
    T, E = weights.shape
    _dev(x, "x", None, (T, x.shape[1]))
    if x.shape[1] % E:
        raise HipLibraryError("the row must hold a whole number of columns an expert")
    _dev(weights, "weights", torch.float32)
    _dev(out, "out", None, tuple(x.shape))
    _call("alice_scale_columns", x.data_ptr(), dtype_code(x.dtype), weights.data_ptr(), out.data_ptr(), dtype_code(out.dtype),
          T, E, x.shape[1] // E, _stream())


def expert_products_supported(dtype: torch.dtype, width: int, expert_width: int) -> bool:
    """Whether expert_products takes these operands: bfloat16, a width that is a multiple of 8 and experts of a multiple of 32."""
    return dtype == torch.bfloat16 and width >= 8 and width % 8 == 0 and expert_width >= 32 and expert_width % 32 == 0


def expert_products(x: torch.Tensor, weights: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, y: torch.Tensor, *,
                    expert_width: int, top: int, epi_param: float) -> None:
    """The routed feed-forward by grouped products: y[t] = sum over the experts e that token t uses (weights[t, e] > 0) of
    weights[t, e] * down_e(act(gate_e x[t]) * (up_e x[t])).  x: bfloat16 [T, W]; weights: float32 [T, E]; gate_up, down: the
    fragment layouts of [all gates; all ups] ([2 E F, W]) and of the down matrices side by side ([W, E F]); y: float32
    [T, W].  The (token, expert) pairs are put in expert order on the device; only the chosen experts are read."""
    T, W = x.shape
    E, F = weights.shape[1], int(expert_width)
    if not expert_products_supported(x.dtype, W, F):
        raise HipLibraryError("expert_products: bfloat16, a width that is a multiple of 8 and experts of a multiple of 32")
    _dev(x, "x", torch.bfloat16)
    _dev(weights, "weights", torch.float32, (T, E))
    _dev(gate_up, "gate_up", torch.bfloat16, (frag_rows(2 * E * F) * (-(-W // 32) * 32),))
    _dev(down, "down", torch.bfloat16, (frag_rows(W) * (-(-(E * F) // 32) * 32),))
    _dev(y, "y", torch.float32, (T, W))
    R = library().alice_expert_rows(T, E, int(top))
    ints = torch.empty((2 * R + R // 64 + T * top,), dtype=torch.int32, device=x.device)
    mid = torch.empty((R, F), dtype=torch.bfloat16, device=x.device)
    rows = torch.empty((R, W), dtype=torch.float32, device=x.device)
    _call("alice_expert_products", x.data_ptr(), weights.data_ptr(), gate_up.data_ptr(), down.data_ptr(), y.data_ptr(),
          ints.data_ptr(), mid.data_ptr(), rows.data_ptr(), T, W, F, E, int(top), float(epi_param), _stream())


def fragment_layout_supported(rows: int, k_in: int, epilogue: int) -> bool:
    """Whether the MFMA kernels take a weight of `rows` x k_in with this epilogue in the fragment layout."""
    return bool(library().alice_frag16_supported(int(rows), int(k_in), int(epilogue)))


KV_ROW, KV_FRAGMENT = 0, 1
ATTN_PARTS_HEAD = 4             # floats before a split's output in the parts of attention_decode (ALICE_ATTN_PARTS_HEAD)
KV_FRAGMENT_PAGE = 64            # positions per page that the fragment layout of keys and values is written for
ATTENTION_MAX_HEAD_DIM = 256     # the largest head size any attention kernel here takes


def attention_mfma_supported(head_dim: int) -> bool:
    """Whether the matrix-core attention kernels (and the fragment cache layout) cover this head size."""
    return bool(library().alice_attention_mfma_supported(int(head_dim)))


def decode_splits(n_seqs: int, num_kv_heads: int, max_context: int) -> int:
    """Into how many blocks the keys of a sequence are split for single-token attention.  At most as many as fill
    the chip (about a thousand waves); among those, the fewest that leave a wave the fewest 32-key blocks to walk
    through one after the other, but no fewer than two (125 blocks of keys: 16 splits of four waves walk two each,
    15 splits three)."""
    n_blocks = -(-max_context // 32)
    cap = max(1, min(-(-1024 // max(1, n_seqs * num_kv_heads * 4)), 64))
    best, best_per = 1, -(-n_blocks // 4)
    for s in range(2, cap + 1):
        per = -(-n_blocks // (4 * s))
        if 2 <= per < best_per:
            best, best_per = s, per
    return best


PREFILL_AUTO, PREFILL_TILES, PREFILL_SPLIT, PREFILL_SHARED4, PREFILL_SHARED8, PREFILL_SHARED4X2 = 0, 1, 2, 3, 4, 5


def attention_prefill(q, k_pool, v_pool, out, cu_seqlens, context_lens, block_table, *, num_heads: int, n_seqs: int,
                      max_new: int, max_context: int, scale: float, softcap: Optional[float], window: Optional[int],
                      variant: int = PREFILL_AUTO, out_layout: int = LAYOUT_ROW) -> None:
    """Prompt attention on the matrix cores.  variant: whole query tiles per wave; one tile's keys split over a
    block's four waves (what fills the chip when there are few tiles); or the four or eight waves of a block
    sharing each block of keys and values through LDS.  AUTO picks by the grid's size.
    out_layout FRAG16: `out` is a flat buffer of ceil16(T) * num_heads * d elements in fragment order."""
    n_pages, nKV, page_size, d = k_pool.shape
    T = q.shape[0]
    _dev(q, "q", torch.bfloat16, (T, num_heads * d))
    if out_layout == LAYOUT_FRAG16:
        _dev(out, "out", torch.bfloat16, (frag_rows(T) * num_heads * d,))
    else:
        _dev(out, "out", torch.bfloat16, (T, num_heads * d))
    _dev(k_pool, "k_pool", torch.bfloat16)
    _dev(v_pool, "v_pool", torch.bfloat16, k_pool.shape)
    _dev(cu_seqlens, "cu_seqlens", torch.int32, (n_seqs + 1,))
    _dev(context_lens, "context_lens", torch.int32, (n_seqs,))
    _dev(block_table, "block_table", torch.int32)
    if block_table.dim() != 2 or block_table.shape[0] < n_seqs or (max_context - 1) // page_size >= block_table.shape[1]:
        raise HipLibraryError(f"{max_context} keys are beyond the block table {tuple(block_table.shape)}")
    _call("alice_attention_prefill", q.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), out.data_ptr(),
          cu_seqlens.data_ptr(), context_lens.data_ptr(), block_table.data_ptr(), block_table.shape[1], n_seqs,
          max_new, num_heads, nKV, d, page_size, float(scale), float(softcap or 0.0), int(window or 0), int(variant),
          int(out_layout), _stream())


def attention_decode(q, k_pool, v_pool, out, context_lens, block_table, *, num_heads: int, max_context: int,
                     scale: float, softcap: Optional[float], window: Optional[int], splits: Optional[int] = None,
                     out_layout: int = LAYOUT_ROW, gate: Optional[torch.Tensor] = None):
    """gate: bfloat16 [B, >= heads] with unit column stride; applied where the key splits are combined (so only with
    splits > 1 and an output; returns False in the third place otherwise and the caller gates the output itself).
    out_layout FRAG16: `out` is a flat buffer of ceil16(B) * num_heads * d elements in fragment order.
    Returns (parts, splits).  With out=None the keys' splits are left uncombined in `parts`
    ([B, heads, splits, 4 + d] float32, flat) for linear_parts(); that needs splits > 1."""
    n_pages, nKV, page_size, d = k_pool.shape
    B = q.shape[0]
    _dev(q, "q", torch.bfloat16, (B, num_heads * d))
    if out is None:
        pass
    elif out_layout == LAYOUT_FRAG16:
        _dev(out, "out", torch.bfloat16, (frag_rows(B) * num_heads * d,))
    else:
        _dev(out, "out", torch.bfloat16, (B, num_heads * d))
    _dev(k_pool, "k_pool", torch.bfloat16)
    _dev(v_pool, "v_pool", torch.bfloat16, k_pool.shape)
    _dev(context_lens, "context_lens", torch.int32, (B,))
    _dev(block_table, "block_table", torch.int32)
    if block_table.dim() != 2 or block_table.shape[0] < B or (max_context - 1) // page_size >= block_table.shape[1]:
        raise HipLibraryError(f"{max_context} keys are beyond the block table {tuple(block_table.shape)}")
    if splits is None:
        reach = max_context if not window else min(max_context, window + 32)
        splits = decode_splits(B, nKV, reach)
    if out is None and splits < 2:
        raise HipLibraryError("attention_decode: without an output buffer the keys must be split")
    parts = (torch.empty((library().alice_attention_decode_workspace(B, num_heads, d, splits),), dtype=torch.float32,
                         device=q.device) if splits > 1 else None)
    gate_ptr, gate_stride = None, 0
    if gate is not None and splits > 1 and out is not None:
        if (not gate.is_cuda or gate.dtype != torch.bfloat16 or gate.dim() != 2 or gate.shape[0] != B
                or gate.shape[1] < num_heads or gate.stride(1) != 1 or gate.stride(0) < num_heads):
            raise HipLibraryError(f"gate must be [{B}, >= {num_heads}] bfloat16 with unit column stride")
        gate_ptr, gate_stride = gate.data_ptr(), gate.stride(0)
    _call("alice_attention_decode", q.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), None if out is None else out.data_ptr(),
          _opt(parts, "parts"), context_lens.data_ptr(), block_table.data_ptr(), block_table.shape[1], B, num_heads,
          nKV, d, page_size, float(scale), float(softcap or 0.0), int(window or 0), splits, int(out_layout),
          gate_ptr, int(gate_stride), _stream())
    if gate is not None:
        return parts, splits, gate_ptr is not None
    return parts, splits


def decode_attention_splits(n_seqs: int, num_kv_heads: int, max_context: int, window: Optional[int]) -> int:
    """The number of key splits that attention_decode picks by itself for a step."""
    reach = max_context if not window else min(max_context, window + 32)
    return decode_splits(n_seqs, num_kv_heads, reach)


def linear_parts_slices(M: int, n_out: int, num_heads: int, head_dim: int, splits: int) -> int:
    """Into how many slices linear_parts() cuts the inner dimension for these sizes; 0 where it does not cover them."""
    return library().alice_linear_parts_split(int(M), int(n_out), int(num_heads), int(head_dim), int(splits))


def linear_parts(parts: torch.Tensor, splits: int, w: torch.Tensor, y: torch.Tensor, *, num_heads: int, head_dim: int) -> None:
    """y[slices, M, n_out] (float32 partial sums) = the output projection of what the uncombined parts of
    attention_decode combine to, without a kernel for the combine: w is the fragment layout of [n_out, heads * d]."""
    if y.dim() != 3:
        raise HipLibraryError("y must be [slices, M, n_out]")
    slices, M, n_out = y.shape
    _dev(y, "y", torch.float32)
    _dev(parts, "parts", torch.float32, (M * num_heads * splits * (ATTN_PARTS_HEAD + head_dim),))
    _dev(w, "w", torch.bfloat16)
    need = ((n_out + 15) // 16 * 16) * (num_heads * head_dim)
    if w.numel() != need:
        raise HipLibraryError(f"w in fragment layout must hold {need} elements, found {w.numel()}")
    if slices != linear_parts_slices(M, n_out, num_heads, head_dim, splits) or slices == 0:
        raise HipLibraryError(f"y must have {linear_parts_slices(M, n_out, num_heads, head_dim, splits)} slices for these sizes (0: not covered)")
    _call("alice_linear_parts", parts.data_ptr(), int(splits), int(num_heads), int(head_dim), w.data_ptr(), y.data_ptr(),
          int(M), int(n_out), _stream())


def attention(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, out: torch.Tensor, ctx,
              block_table: torch.Tensor, *, num_heads: int, scale: float, softcap: Optional[float],
              window: Optional[int], full_precision: bool, kv_layout: int = KV_ROW,
              out_layout: int = LAYOUT_ROW, bias_slopes: Optional[torch.Tensor] = None,
              gate: Optional[torch.Tensor] = None) -> None:
    """Attention of the step's query tokens over the cache; picks the kernel for the step's shape and
    the cache's layout.  `ctx` carries positions, seq_of_token, cu_seqlens, context_lens and the
    host-side sizes of the step.  out_layout FRAG16 is taken by the matrix-core kernels only; a score bias
    (bias_slopes, see attention_generic) by the generic kernel only, over a row-major cache."""
    if kv_layout == KV_FRAGMENT:
        if bias_slopes is not None:
            raise HipLibraryError("the matrix-core attention kernels take no score bias: lay the cache out row-major")
        nKV = k_pool.shape[1]
        if ctx.is_decode and num_heads // nKV <= 16:
            res = attention_decode(q, k_pool, v_pool, out, ctx.context_lens, block_table, num_heads=num_heads,
                                   max_context=ctx.max_context, scale=scale, softcap=softcap, window=window,
                                   out_layout=out_layout, gate=gate)
            if gate is not None and res[2]:
                return                                         # gated where the key splits were combined
        else:
            attention_prefill(q, k_pool, v_pool, out, ctx.cu_seqlens, ctx.context_lens, block_table,
                              num_heads=num_heads, n_seqs=ctx.n_seqs, max_new=ctx.max_new,
                              max_context=ctx.max_context, scale=scale, softcap=softcap, window=window,
                              out_layout=out_layout)
        if gate is not None:
            head_gate(out, out_layout, gate, q.shape[0], num_heads, k_pool.shape[3])
        return
    if out_layout != LAYOUT_ROW:
        raise HipLibraryError("only the matrix-core attention kernels write fragment order")
    attention_generic(q, k_pool, v_pool, out, ctx.positions, ctx.seq_of_token, block_table,
                      num_heads=num_heads, scale=scale, softcap=softcap, window=window,
                      max_position=ctx.max_position, full_precision=full_precision, bias_slopes=bias_slopes, gate=gate)


MLSTM_MAX_VALUE_DIM = 1024      # the largest value head size the matrix-memory kernels take


def mlstm(proj, bias_i, bias_f, norm_w, out, ctx, S, n, m, *, heads: int, head_dim: int, value_head_dim: int,
          cap: float, eps: float) -> None:
    """The matrix memory over a step: `ctx` carries cu_seqlens, slots and the host-side sizes (see mlstm_rows)."""
    mlstm_rows(proj, bias_i, bias_f, norm_w, out, ctx.cu_seqlens, ctx.slots, S, n, m, n_seqs=ctx.n_seqs,
               max_new=ctx.max_new, heads=heads, head_dim=head_dim, value_head_dim=value_head_dim, cap=cap, eps=eps)


def mlstm_rows(proj, bias_i, bias_f, norm_w, out, cu_seqlens, slots, S, n, m, *, n_seqs: int, max_new: int, heads: int,
               head_dim: int, value_head_dim: int, cap: float, eps: float) -> None:
    """Picks the kernel for the step's shape: token by token for single tokens and pieces of a few tokens, a chunk
    of tokens at a time on the matrix cores for longer ones (head sizes that are multiples of 16, keys up to 256)."""
    if (max_new >= MLSTM_CHUNK_FROM and proj.shape[1] % 4 == 0
            and library().alice_mlstm_chunks_supported(int(n_seqs), heads, head_dim, value_head_dim)):
        mlstm_chunks(proj, bias_i, bias_f, norm_w, out, cu_seqlens, slots, S, n, m, n_seqs=n_seqs, heads=heads,
                     head_dim=head_dim, value_head_dim=value_head_dim, cap=cap, eps=eps, max_new=max_new)
        return
    if head_dim <= MLSTM_COLS_MAX_KEY_DIM:
        mlstm_chunks(proj, bias_i, bias_f, norm_w, out, cu_seqlens, slots, S, n, m, n_seqs=n_seqs, heads=heads,
                     head_dim=head_dim, value_head_dim=value_head_dim, cap=cap, eps=eps, entry="alice_mlstm_cols")
        return
    mlstm_step(proj, bias_i, bias_f, norm_w, out, cu_seqlens, slots, S, n, m, n_seqs=n_seqs, heads=heads,
               head_dim=head_dim, value_head_dim=value_head_dim, cap=cap, eps=eps)


MLSTM_COLS_MAX_KEY_DIM = 256      # key sizes up to this keep the state in registers over a step (alice_mlstm_cols)
MLSTM_CHUNK_FROM = 4      # steps whose longest piece has at least this many tokens take the chunk kernel


def _mlstm_args(proj, bias_i, bias_f, norm_w, out, cu_seqlens, slots, S, n, m, n_seqs, H, d, dv):
    T = proj.shape[0]
    _dev(proj, "proj", torch.float32)
    if proj.dim() != 2 or proj.shape[1] < 2 * H * d + 2 * H * dv + 2 * H:
        raise HipLibraryError(f"proj rows of {tuple(proj.shape)} are too short")
    _dev(bias_i, "bias_i", torch.float32, (H,))
    _dev(bias_f, "bias_f", torch.float32, (H,))
    _dev(norm_w, "norm_w", None, (H * dv,))
    _dev(out, "out", None, (T, H * dv))
    _dev(cu_seqlens, "cu_seqlens", torch.int32)
    _dev(slots, "slots", torch.int32)
    if cu_seqlens.numel() < n_seqs + 1 or slots.numel() < n_seqs:
        raise HipLibraryError("cu_seqlens and slots are too short for the step's sequences")
    n_slots = S.shape[0]
    _dev(S, "S", torch.float32, (n_slots, H, d, dv))
    _dev(n, "n", torch.float32, (n_slots, H, d))
    _dev(m, "m", torch.float32, (n_slots, H))
    return T, n_slots


def mlstm_chunks(proj, bias_i, bias_f, norm_w, out, cu_seqlens, slots, S, n, m, *, n_seqs: int, heads: int, head_dim: int,
                 value_head_dim: int, cap: float, eps: float, entry: str = "alice_mlstm_chunks",
                 max_new: Optional[int] = None) -> None:
    """mlstm_step's result by the chunk kernel, or with entry="alice_mlstm_cols" by the kernel of single tokens
    (see mlstm.hip); allocates their float32 workspace [T, H dv]."""
    H, d, dv = heads, head_dim, value_head_dim
    T, n_slots = _mlstm_args(proj, bias_i, bias_f, norm_w, out, cu_seqlens, slots, S, n, m, n_seqs, H, d, dv)
    args = [proj.data_ptr(), proj.shape[1], bias_i.data_ptr(), bias_f.data_ptr(), norm_w.data_ptr(), dtype_code(norm_w.dtype),
            out.data_ptr(), dtype_code(out.dtype)]
    tail = [cu_seqlens.data_ptr(), slots.data_ptr(), S.data_ptr(), n.data_ptr(), m.data_ptr(), T, int(n_seqs), int(n_slots),
            H, d, dv, float(cap), float(eps)]
    if entry == "alice_mlstm_chunks":
        # read-outs, denominators and, where the chunks run side by side, every chunk's state; max_new: the most
        # tokens of one sequence (the whole step's where the caller does not say)
        max_new = T if max_new is None else max(1, min(int(max_new), T))
        work = torch.empty((library().alice_mlstm_chunks_workspace(T, int(n_seqs), max_new, H, d, dv),), dtype=torch.float32,
                           device=proj.device)
        _call(entry, *args, work.data_ptr(), *tail, max_new, _stream())
    else:
        work = torch.empty((T, H * dv), dtype=torch.float32, device=proj.device)
        _call(entry, *args, work.data_ptr(), *tail, _stream())


def mlstm_step(proj: torch.Tensor, bias_i: torch.Tensor, bias_f: torch.Tensor, norm_w: torch.Tensor, out: torch.Tensor,
               cu_seqlens: torch.Tensor, slots: torch.Tensor, S: torch.Tensor, n: torch.Tensor, m: torch.Tensor, *,
               n_seqs: int, heads: int, head_dim: int, value_head_dim: int, cap: float, eps: float) -> None:
    """The matrix memory over the step's tokens, sequence by sequence from the state rows slots[s], with the head
    norm, its weight and the output gate behind it.  proj: float32 [T, >= 2 H d + 2 H dv + 2 H] rows
    [q | k | v | g | a | b]; out: [T, H dv] in the activation dtype; S [slots, H, d, dv], n [slots, H, d],
    m [slots, H] float32."""
    H, d, dv = heads, head_dim, value_head_dim
    T = proj.shape[0]
    _dev(proj, "proj", torch.float32)
    if proj.dim() != 2 or proj.shape[1] < 2 * H * d + 2 * H * dv + 2 * H:
        raise HipLibraryError(f"proj rows of {tuple(proj.shape)} are too short")
    _dev(bias_i, "bias_i", torch.float32, (H,))
    _dev(bias_f, "bias_f", torch.float32, (H,))
    _dev(norm_w, "norm_w", None, (H * dv,))
    _dev(out, "out", None, (T, H * dv))
    _dev(cu_seqlens, "cu_seqlens", torch.int32)
    _dev(slots, "slots", torch.int32)
    if cu_seqlens.numel() < n_seqs + 1 or slots.numel() < n_seqs:
        raise HipLibraryError("cu_seqlens and slots are too short for the step's sequences")
    n_slots = S.shape[0]
    _dev(S, "S", torch.float32, (n_slots, H, d, dv))
    _dev(n, "n", torch.float32, (n_slots, H, d))
    _dev(m, "m", torch.float32, (n_slots, H))
    _call("alice_mlstm_step", proj.data_ptr(), proj.shape[1], bias_i.data_ptr(), bias_f.data_ptr(), norm_w.data_ptr(),
          dtype_code(norm_w.dtype), out.data_ptr(), dtype_code(out.dtype), cu_seqlens.data_ptr(), slots.data_ptr(),
          S.data_ptr(), n.data_ptr(), m.data_ptr(), int(n_seqs), int(n_slots), H, d, dv, float(cap), float(eps), _stream())


def gelu_mul_rows(z: torch.Tensor, table: torch.Tensor, col0: int, tokens: torch.Tensor, out: torch.Tensor, *,
                  full_precision: bool) -> None:
    """out[t, j] = gelu_tanh(z[t, j]) * table[tokens[t], col0 + j]; table: row-major [V, width]."""
    T, n = z.shape
    _dev(z, "z")
    _dev(out, "out", z.dtype, (T, n))
    _dev(tokens, "tokens", torch.int32)
    if tokens.numel() < T or table.dim() != 2:
        raise HipLibraryError("gelu_mul_rows: one token per row and a [V, width] table")
    _dev(table, "table")
    _call("alice_gelu_mul_rows", z.data_ptr(), dtype_code(z.dtype), table.data_ptr(), dtype_code(table.dtype), table.shape[1],
          int(col0), tokens.data_ptr(), out.data_ptr(), dtype_code(out.dtype), T, n, table.shape[0], int(full_precision), _stream())


def head_gate(out: torch.Tensor, out_layout: int, gate: torch.Tensor, T: int, num_heads: int, head_dim: int) -> None:
    """out[t, h, :] *= sigmoid(gate[t, h]) in place; out: bfloat16 [T, heads * d] row-major, or its flat fragment
    order; gate: bfloat16 [T, >= heads] with unit column stride (a column slice of a wider tensor)."""
    if out_layout == LAYOUT_FRAG16:
        _dev(out, "out", torch.bfloat16, (frag_rows(T) * num_heads * head_dim,))
    else:
        _dev(out, "out", torch.bfloat16, (T, num_heads * head_dim))
    if (not gate.is_cuda or gate.dtype != torch.bfloat16 or gate.dim() != 2 or gate.shape[0] != T
            or gate.shape[1] < num_heads or gate.stride(1) != 1 or gate.stride(0) < num_heads):
        raise HipLibraryError(f"gate must be [{T}, >= {num_heads}] bfloat16 with unit column stride")
    _call("alice_head_gate", out.data_ptr(), int(out_layout), gate.data_ptr(), gate.stride(0), T, num_heads, head_dim, _stream())


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """int32 [B]: index of each row's maximum, the lowest index among equal maxima."""
    _dev(logits, "logits", torch.float32)
    B, V = logits.shape
    if out is None:
        out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    _dev(out, "out", torch.int32, (B,))
    chunks = library().alice_argmax_chunks(B, V)
    wv = wi = None
    if chunks > 1:
        wv = torch.empty((B * chunks,), dtype=torch.float32, device=logits.device)
        wi = torch.empty((B * chunks,), dtype=torch.int32, device=logits.device)
    _call("alice_argmax", logits.data_ptr(), out.data_ptr(), _opt(wv, "work"), _opt(wi, "work"), B, V, _stream())
    return out


_sample_work = {}        # (device, B, V) -> the workspace of sample(): calls on one device's stream follow each other


def sample(logits: torch.Tensor, uniform: torch.Tensor, temperature: float, top_k: int = 0, top_p: float = 1.0,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """int32 [B]: temperature, top-k, top-p, softmax and inverse CDF with uniform[row] in [0, 1)."""
    _dev(logits, "logits", torch.float32)
    B, V = logits.shape
    _dev(uniform, "uniform", torch.float32, (B,))
    if out is None:
        out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    _dev(out, "out", torch.int32, (B,))
    key = (logits.device, B, V)
    work = _sample_work.get(key)
    if work is None:
        if len(_sample_work) > 16:
            _sample_work.clear()
        work = _sample_work[key] = torch.empty((library().alice_sample_workspace(B, V) + 1) // 2, dtype=torch.int64,
                                               device=logits.device)
    _call("alice_sample", logits.data_ptr(), out.data_ptr(), uniform.data_ptr(), work.data_ptr(), B, V,
          float(temperature), int(top_k), float(top_p), _stream())
    return out
