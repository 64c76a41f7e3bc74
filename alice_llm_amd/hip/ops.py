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
ABI_VERSION = 6

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
        "alice_linear": [P, I, P, I, I, P, I, I, I, I, I, F, I, I, I, I, I, P],
        "alice_linear_split_hint": [I, I, I, I],
        "alice_to_frag16": [P, P, I, I, P],
        "alice_frag16_supported": [I, I, I],
        "alice_rope_cache_write": [P, I, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I, I, I, P],
        "alice_linear_rope_cache": [P, I, P, I, I, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, P],
        "alice_attention_mfma_supported": [I],
        "alice_attention_prefill": [P, P, P, P, P, P, P, I, I, I, I, I, I, I, F, F, I, I, I, P],
        "alice_attention_decode": [P, P, P, P, P, P, P, I, I, I, I, I, I, F, F, I, I, I, P],
        "alice_attention_generic": [P, I, P, P, P, P, P, P, I, I, I, I, I, I, F, F, I, P, I, P],
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
                     rotary_dim: int, max_position: int, kv_layout: int = 0, interleaved: bool = False) -> None:
    """Rotate q and k; write k and v at their positions into the pools [pages, nKV, page, d].
    With k_pool None the row holds q only (num_kv_heads = 0) and nothing is cached.
    `max_position` is the largest position among `positions` (the host knows it): checked against the tables.
    interleaved: the q and k heads of qkv hold the rotated pairs (j, j + d/2) at 2j and 2j + 1 (a projection
    with its rows in that order made them); the outputs are in the plain order either way."""
    T = qkv.shape[0]
    dt = qkv.dtype
    _dev(qkv, "qkv")
    row_width = qkv.shape[1]
    if qkv.dim() != 2 or row_width < (num_heads + (2 * num_kv_heads if k_pool is not None else 0)) * head_dim:
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
        _dev(v_pool, "v_pool", dt, k_pool.shape)
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
          num_kv_heads, head_dim, rotary_dim, page_size, n_pages, int(kv_layout), int(interleaved), _stream())


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
                      max_position: int, full_precision: bool, bias_slopes: Optional[torch.Tensor] = None) -> None:
    """bias_slopes: float32 [num_heads]; head h's capped score of key k for the query at position p gets
    bias_slopes[h] * (k - p) added before the softmax."""
    T = q.shape[0]
    dt = q.dtype
    if k_pool.dim() != 4:
        raise HipLibraryError("k_pool must be [pages, nKV, page, d]")
    n_pages, nKV, page_size, d = k_pool.shape
    _dev(q, "q", None, (T, num_heads * d))
    _dev(out, "out", dt, (T, num_heads * d))
    _dev(k_pool, "k_pool", dt)
    _dev(v_pool, "v_pool", dt, k_pool.shape)
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
          int(full_precision), _stream())


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
                     out_layout: int = LAYOUT_ROW):
    """out_layout FRAG16: `out` is a flat buffer of ceil16(B) * num_heads * d elements in fragment order.
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
    _call("alice_attention_decode", q.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), None if out is None else out.data_ptr(),
          _opt(parts, "parts"), context_lens.data_ptr(), block_table.data_ptr(), block_table.shape[1], B, num_heads,
          nKV, d, page_size, float(scale), float(softcap or 0.0), int(window or 0), splits, int(out_layout), _stream())
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
              out_layout: int = LAYOUT_ROW, bias_slopes: Optional[torch.Tensor] = None) -> None:
    """Attention of the step's query tokens over the cache; picks the kernel for the step's shape and
    the cache's layout.  `ctx` carries positions, seq_of_token, cu_seqlens, context_lens and the
    host-side sizes of the step.  out_layout FRAG16 is taken by the matrix-core kernels only; a score bias
    (bias_slopes, see attention_generic) by the generic kernel only, over a row-major cache."""
    if kv_layout == KV_FRAGMENT:
        if bias_slopes is not None:
            raise HipLibraryError("the matrix-core attention kernels take no score bias: lay the cache out row-major")
        nKV = k_pool.shape[1]
        if ctx.is_decode and num_heads // nKV <= 16:
            attention_decode(q, k_pool, v_pool, out, ctx.context_lens, block_table, num_heads=num_heads,
                             max_context=ctx.max_context, scale=scale, softcap=softcap, window=window,
                             out_layout=out_layout)
            return
        attention_prefill(q, k_pool, v_pool, out, ctx.cu_seqlens, ctx.context_lens, block_table,
                          num_heads=num_heads, n_seqs=ctx.n_seqs, max_new=ctx.max_new,
                          max_context=ctx.max_context, scale=scale, softcap=softcap, window=window,
                          out_layout=out_layout)
        return
    if out_layout != LAYOUT_ROW:
        raise HipLibraryError("only the matrix-core attention kernels write fragment order")
    attention_generic(q, k_pool, v_pool, out, ctx.positions, ctx.seq_of_token, block_table,
                      num_heads=num_heads, scale=scale, softcap=softcap, window=window,
                      max_position=ctx.max_position, full_precision=full_precision, bias_slopes=bias_slopes)


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
