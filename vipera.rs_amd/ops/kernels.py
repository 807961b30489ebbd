"""Python bindings of the HIP kernels: shape checks on the host, then one launch on the current stream.

Every function takes device tensors, checks that their shapes and dtypes are what the kernel
and its grid assume, and launches on ``torch.cuda.current_stream()``.  There is no fallback:
when a library cannot be built or loaded the call raises.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..errors import InternalError, InvalidArgumentError, UnsupportedError
from .build import load_module

_DT = {torch.float32: 0, torch.bfloat16: 1}
_p = ctypes.c_void_p
_i = ctypes.c_int
_ll = ctypes.c_longlong
_f = ctypes.c_float


def _dt(tensor: torch.Tensor, what: str) -> int:
    if tensor.dtype not in _DT:
        raise UnsupportedError(f"{what} has dtype {tensor.dtype}; float32 and bfloat16 are implemented")
    return _DT[tensor.dtype]


def _ptr(tensor: Optional[torch.Tensor]):
    return _p(tensor.data_ptr()) if tensor is not None else _p(0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current stream's handle.  Through torch's raw accessors where it has them: ``torch.cuda.current_stream()``
    builds a Python object on every call, which was a quarter of the host's time for a step launched kernel by kernel."""
    if _raw_stream is not None and _raw_device is not None:
        return _p(_raw_stream(_raw_device()))
    return _p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, text: str) -> None:
    if not cond:
        raise InvalidArgumentError(text)


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for tensor in tensors:
        if tensor is not None and not tensor.is_cuda:
            raise InvalidArgumentError("kernel operands must live on the GPU; got a CPU tensor")


def _status(code: int, name: str) -> None:
    if code == 0:
        return
    if code == -1:
        raise InvalidArgumentError(f"{name}: the launcher refused its arguments")
    if code == -2:
        raise UnsupportedError(f"{name}: a size is outside what this kernel is built for")
    raise InternalError(f"{name}: HIP error {code} at launch")


ATTENTION_MAX_HEAD_DIM = 256    # both attention kernels keep a head's dims in registers or one LDS row
ATTENTION_MAX_HEADS = 65_535    # q, k and v heads of a token are one grid dimension of the rotation kernel
GEMM_BF16_MAX_K = 1 << 23       # the matrix-core products form 32-bit byte offsets inside a tile of rows


def _cache_ok(k_cache, v_cache, kv_heads: int, head_dim: int, dtype) -> bool:
    """K pages ``[pages, kv_heads, block_size, head_dim]``, V pages ``[pages, kv_heads, head_dim, block_size]``."""
    return (k_cache.dim() == 4 and v_cache.dim() == 4 and k_cache.shape[1] == kv_heads
            and k_cache.shape[3] == head_dim and v_cache.shape[1] == kv_heads and v_cache.shape[2] == head_dim
            and v_cache.shape[0] == k_cache.shape[0] and v_cache.shape[3] == k_cache.shape[2]
            and k_cache.dtype == dtype and v_cache.dtype == dtype and k_cache.is_contiguous()
            and v_cache.is_contiguous())


_signatures_done = set()


def _fn(module: str, name: str, argtypes, key: str = None):
    library = load_module(module)
    fn = getattr(library, name)
    key = key or name
    if key not in _signatures_done:
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
        _signatures_done.add(key)
    return fn


# ----------------------------------------------------------------------------------------------
def fetch_words(pinned: torch.Tensor, out: torch.Tensor) -> bool:
    """``out[:] = pinned[:]`` (int32 words) by a kernel that reads the pinned host tensor directly, in the current
    stream.  Returns False, having done nothing, if the runtime does not give the host memory a device address
    (the caller then copies with ``out.copy_``)."""
    _dev(out)
    _need(not pinned.is_cuda and pinned.is_pinned(), "fetch_words: the source must be pinned host memory")
    _need(pinned.dtype == torch.int32 and out.dtype == torch.int32 and pinned.is_contiguous() and out.is_contiguous()
          and pinned.numel() == out.numel(), "fetch_words: two contiguous int32 tensors of one size")
    fn = _fn("elementwise", "vk_fetch_words", [_p, _p, _ll, _p])
    code = fn(pinned.data_ptr(), _ptr(out), out.numel(), _stream())
    if code == -2:
        return False
    _status(code, "fetch_words")
    return True


# ----------------------------------------------------------------------------------------------
def embed_gather(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor,
                 source: Optional[torch.Tensor] = None, sampled: Optional[torch.Tensor] = None) -> None:
    """``out[t, :] = table[tokens[t], :]`` widened to 32-bit.  The caller has checked the ids.

    With ``source`` and ``sampled``: where ``source[t] >= 0`` the id is ``sampled[source[t]]``, which an
    earlier kernel of the stream left on the device."""
    _dev(table, tokens, out, source, sampled)
    num_tokens, width = out.shape
    _need(table.dim() == 2 and table.shape[1] == width and table.is_contiguous(), "embed_gather: table shape")
    _need(tokens.dtype == torch.int32 and tokens.numel() >= num_tokens and tokens.is_contiguous(), "embed_gather: tokens")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "embed_gather: out must be contiguous float32")
    if source is not None:
        _need(sampled is not None and sampled.dtype == torch.int32 and sampled.is_contiguous(),
              "embed_gather: sampled must be contiguous int32")
        _need(source.dtype == torch.int32 and source.numel() >= num_tokens and source.is_contiguous(),
              "embed_gather: source")
    fn = _fn("elementwise", "vk_embed_gather", [_p, _i, _p, _p, _p, _p, _i, _i, _i, _p])
    _status(fn(_ptr(table), _dt(table, "table"), _ptr(tokens), _ptr(source), _ptr(sampled if source is not None else None),
               _ptr(out), num_tokens, width, table.shape[0], _stream()), "embed_gather")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            rows: Optional[torch.Tensor] = None) -> None:
    """``out[r] = x[rows[r]] * rsqrt(mean(x^2) + eps) * weight`` (``rows`` absent: every row in order)."""
    _dev(x, weight, out, rows)
    num_rows, width = out.shape
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.shape[1] == width and x.is_contiguous(), "rmsnorm: x")
    _need(weight.dtype == torch.float32 and weight.numel() == width and weight.is_contiguous(), "rmsnorm: weight")
    _need(out.is_contiguous(), "rmsnorm: out must be contiguous")
    if rows is None:
        _need(x.shape[0] >= num_rows, "rmsnorm: fewer input rows than output rows")
    else:
        _need(rows.dtype == torch.int32 and rows.numel() >= num_rows and rows.is_contiguous(), "rmsnorm: rows")
    fn = _fn("elementwise", "vk_rmsnorm", [_p, _p, _p, _p, _i, _i, _i, _f, _p])
    _status(fn(_ptr(x), _ptr(weight), _ptr(rows), _ptr(out), _dt(out, "out"), num_rows, width, float(eps), _stream()),
            "rmsnorm")


def rope_angles(positions: torch.Tensor, inv_freq: torch.Tensor, num_tokens: int) -> torch.Tensor:
    """``[num_tokens, len(inv_freq), 2]`` floats: sine and cosine of ``float(pos) * inv_freq`` for a step's
    tokens, computed once where many heads and layers would each compute them again."""
    _dev(positions, inv_freq)
    _need(positions.dtype == torch.int32 and positions.numel() >= num_tokens, "rope_angles: positions")
    _need(inv_freq.dtype == torch.float32 and inv_freq.is_contiguous(), "rope_angles: inv_freq must be float32")
    out = torch.empty((num_tokens, inv_freq.numel(), 2), dtype=torch.float32, device=positions.device)
    fn = _fn("elementwise", "vk_rope_angles", [_p, _p, _i, _i, _p, _p])
    _status(fn(_ptr(positions), _ptr(inv_freq), inv_freq.numel(), num_tokens, _ptr(out), _stream()), "rope_angles")
    return out


def rope_kvwrite(qkv: torch.Tensor, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rotary_dim: int,
                 k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], entry_of_token: torch.Tensor,
                 block_table: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int,
                 angles: Optional[torch.Tensor] = None) -> None:
    """Rotate the q and k heads of ``qkv`` in place, then store the tokens' K and V in their pages.
    ``angles``: the step's table from :func:`rope_angles`, used instead of computing sines and cosines here.

    ``k_cache``: ``[pages, kv_heads, block_size, head_dim]``; ``v_cache`` is transposed,
    ``[pages, kv_heads, head_dim, block_size]``; ``block_table``: ``[entries, width]``.
    The caller guarantees that every token's page exists in its entry's row of the table.
    """
    _dev(qkv, positions, inv_freq, k_cache, v_cache, entry_of_token, block_table)
    num_tokens = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (heads + 2 * kv_heads) * head_dim and qkv.is_contiguous(),
          "rope_kvwrite: qkv must be [tokens, (heads + 2 kv_heads) * head_dim]")
    _need(positions.dtype == torch.int32 and positions.numel() >= num_tokens, "rope_kvwrite: positions")
    _need(0 <= rotary_dim <= head_dim and rotary_dim % 2 == 0, "rope_kvwrite: rotary_dim")
    if rotary_dim:
        _need(inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() == rotary_dim // 2,
              "rope_kvwrite: inv_freq must hold rotary_dim / 2 floats")
    table_width = block_size = 0
    if k_cache is not None:
        _need(v_cache is not None and block_table is not None, "rope_kvwrite: cache without table")
        _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, qkv.dtype), "rope_kvwrite: cache shape or dtype")
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
              "rope_kvwrite: block table")
        _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() >= num_tokens, "rope_kvwrite: entries")
        table_width, block_size = block_table.shape[1], k_cache.shape[2]
    if angles is not None:
        _dev(angles)
        _need(rotary_dim > 0 and angles.dtype == torch.float32 and angles.is_contiguous()
              and angles.shape == (num_tokens, rotary_dim // 2, 2), "rope_kvwrite: angles must be [tokens, rotary_dim / 2, 2]")
    fn = _fn("elementwise", "vk_rope_kvwrite", [_p, _i, _p, _p, _p, _i, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p])
    _status(fn(_ptr(qkv), _dt(qkv, "qkv"), _ptr(positions), _ptr(inv_freq), _ptr(angles), rotary_dim, _ptr(k_cache), _ptr(v_cache),
               _ptr(entry_of_token), _ptr(block_table), table_width, block_size, num_tokens, heads, kv_heads,
               head_dim, _stream()), "rope_kvwrite")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, interleaved: bool = False) -> None:
    """``out = up * silu(gate)``; a row of ``gate_up`` is ``[gate | up]``, or with ``interleaved`` groups of
    16 gate columns followed by the 16 up columns of the same outputs."""
    _dev(gate_up, out)
    num_tokens, inter = out.shape
    _need(gate_up.shape == (num_tokens, 2 * inter) and gate_up.dtype == out.dtype and gate_up.is_contiguous()
          and out.is_contiguous(), "swiglu: gate_up must be [tokens, 2 * intermediate] of out's dtype")
    _need(not interleaved or inter % 16 == 0, "swiglu: the interleaved layout needs a multiple of 16 outputs")
    fn = _fn("elementwise", "vk_swiglu", [_p, _p, _i, _i, _i, _i, _p])
    _status(fn(_ptr(gate_up), _ptr(out), _dt(out, "out"), num_tokens, inter, 1 if interleaved else 0, _stream()), "swiglu")


def fill_normal(out: torch.Tensor, key: int, std: float, offset: float = 0.0) -> None:
    """Fill with ``offset + std * n_i``, ``n_i`` the counter-based normal stream of ``key``."""
    _dev(out)
    _need(out.is_contiguous(), "fill_normal: out must be contiguous")
    fn = _fn("elementwise", "vk_fill_normal", [_p, _i, _ll, ctypes.c_ulonglong, _f, _f, _p])
    _status(fn(_ptr(out), _dt(out, "out"), out.numel(), key & ((1 << 64) - 1), float(std), float(offset), _stream()),
            "fill_normal")


# ----------------------------------------------------------------------------------------------
def gemm_generic(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                 accumulate: bool = False) -> None:
    """``out (+)= a @ w.T + bias`` in 32-bit FMA; ``a`` and ``out`` may be row-strided views."""
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm: operands must be matrices")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n), f"gemm: shapes {tuple(a.shape)} x {tuple(w.shape)}^T -> {tuple(out.shape)}")
    _need(a.stride(1) == 1 and out.stride(1) == 1 and w.is_contiguous(), "gemm: inner strides must be 1")
    _need(a.stride(0) >= k or m == 1, "gemm: a's row stride")
    _need(out.stride(0) >= n or m == 1, "gemm: out's row stride")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    if accumulate:
        _need(out.dtype == torch.float32, "gemm: accumulation needs a float32 output")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n)
    if (m <= 64 and a.dtype == torch.float32 and w.dtype == torch.float32 and k >= 4 and k % 4 == 0 and lda % 4 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and k < 65535 * 1024):
        # up to 64 tokens in 32-bit: a stream of the weights (the same sums in the same order as the tiled kernel)
        slabs = _split_k_workspace(a.device, ((k + 1023) // 1024) * m * n, "stream")
        fn = _fn("gemm_generic", "vk_gemm_stream", [_p, _p, _p, _p, _i, _i, _i, _i, _ll, _ll, _i, _p, _ll, _p])
        _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), _dt(out, "out"), m, n, k, lda, ldc, 1 if accumulate else 0,
                   _ptr(slabs), slabs.numel(), _stream()), "gemm_stream")
        return
    fn = _fn("gemm_generic", "vk_gemm_generic", [_p, _i, _p, _i, _p, _p, _i, _i, _i, _i, _ll, _ll, _i, _p])
    _status(fn(_ptr(a), _dt(a, "a"), _ptr(w), _dt(w, "w"), _ptr(bias), _ptr(out), _dt(out, "out"), m, n, k, lda, ldc,
               1 if accumulate else 0, _stream()), "gemm_generic")


# ----------------------------------------------------------------------------------------------
def attn_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                 positions: torch.Tensor, entry_of_token: torch.Tensor, block_table: torch.Tensor,
                 heads: int, kv_heads: int, head_dim: int, scale: float, window: int,
                 skip_single_of: Optional[torch.Tensor] = None, softcap: float = 0.0, extras=None) -> None:
    """Causal GQA over the paged cache for every token of the step, in 32-bit arithmetic.  ``window`` > 0: the last
    that many positions; < 0: the positions of the token's own block of ``-window`` consecutive positions (counted
    from position 0); ``softcap`` > 0: scores become ``softcap * tanh(score / softcap)`` (all attention kernels alike).

    ``q``: a view ``[tokens, >= heads * head_dim]`` whose row holds the query heads first (the fused
    qkv buffer qualifies); ``out``: ``[tokens, heads * head_dim]``.  ``skip_single_of``: the step's
    ``entry_start``; tokens of entries that hold one token are then left alone (for :func:`attn_decode_f32`).
    """
    _dev(q, k_cache, v_cache, out, positions, entry_of_token, block_table, skip_single_of)
    if skip_single_of is not None:
        _need(skip_single_of.dtype == torch.int32 and skip_single_of.numel() == block_table.shape[0] + 1,
              "attention: entry_start must hold one offset per entry and the end")
    num_tokens = out.shape[0]
    _need(q.dim() == 2 and q.shape[0] == num_tokens and q.stride(1) == 1 and q.shape[1] >= heads * head_dim, "attention: q")
    _need(out.shape == (num_tokens, heads * head_dim) and out.is_contiguous() and out.dtype == q.dtype, "attention: out")
    _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, q.dtype), "attention: cache shape or dtype")
    _need(positions.dtype == torch.int32 and positions.numel() >= num_tokens, "attention: positions")
    _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() >= num_tokens, "attention: entries")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(), "attention: table")
    _need(heads % kv_heads == 0, "attention: heads must be a multiple of kv_heads")
    if head_dim > ATTENTION_MAX_HEAD_DIM:
        raise UnsupportedError(f"attention: head_dim {head_dim} is above the kernels' limit of {ATTENTION_MAX_HEAD_DIM}")
    fn = _fn("attn_generic", "vk_attn_generic_ext",
             [_p, _ll, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _i, _f, _i, _f, _p, _p, _p, _i, _i, _p])
    _status(fn(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _dt(q, "q"), _ptr(positions),
               _ptr(entry_of_token), _ptr(block_table), block_table.shape[1], k_cache.shape[2], num_tokens, heads,
               kv_heads, head_dim, float(scale), int(window), float(softcap), _ptr(skip_single_of),
               *attn_extras_args(extras, heads, window), _stream()), "attn_generic")


def attn_extras_args(extras, heads: int, window: int):
    """``(sink, rel, rel_far, keep_first)`` as the attention launchers take them; ``extras`` (or None) has the
    attributes ``sink`` ([heads] 32-bit or None: a learned logit per head that joins the softmax's denominator only),
    ``rel`` ([heads, rel_far + 1] 32-bit or None: a bias by distance, the last column for every distance from
    ``rel_far`` on) and ``keep_first`` (positions below it stay visible to a windowed layer)."""
    if extras is None:
        return _p(0), _p(0), 0, 0
    sink, rel, keep_first = extras.sink, extras.rel, int(extras.keep_first or 0)
    _dev(sink, rel)
    rel_far = 0
    if sink is not None:
        _need(sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == heads,
              "attention: one 32-bit sink logit per query head")
    if rel is not None:
        _need(rel.dtype == torch.float32 and rel.is_contiguous() and rel.dim() == 2 and rel.shape[0] == heads
              and rel.shape[1] >= 1, "attention: the bias by distance is [heads, distances] in 32-bit")
        rel_far = rel.shape[1] - 1
    _need(keep_first >= 0 and (keep_first == 0 or window > 0), "attention: kept first positions need a window")
    return _ptr(sink), _ptr(rel), rel_far, keep_first


ATTN_DECODE_F32_CHUNK = 256   # positions of one workgroup of attn_decode_f32 (the kernel's DEC_CHUNK)


def attn_decode_f32_supported(q: torch.Tensor, k_cache: torch.Tensor, head_dim: int) -> bool:
    """Whether :func:`attn_decode_f32` takes the operands: all 32-bit, a head width and pages that are multiples
    of 4, 16-byte rows."""
    return (q.dtype == torch.float32 and k_cache.dtype == torch.float32 and head_dim % 4 == 0
            and head_dim <= ATTENTION_MAX_HEAD_DIM and k_cache.shape[2] % 4 == 0 and q.stride(0) % 4 == 0
            and q.data_ptr() % 16 == 0)


def attn_decode_f32(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                    partial: torch.Tensor, entries: torch.Tensor, entry_start: torch.Tensor,
                    entry_first_pos: torch.Tensor, block_table: torch.Tensor, heads: int, kv_heads: int,
                    head_dim: int, scale: float, window: int, chunks: int, softcap: float = 0.0, extras=None) -> None:
    """32-bit attention of the single-token entries listed in ``entries``; their positions are split into
    ``chunks`` of :data:`ATTN_DECODE_F32_CHUNK`, which must cover the longest visible range."""
    _dev(q, k_cache, v_cache, out, partial, entries, entry_start, entry_first_pos, block_table)
    _need(attn_decode_f32_supported(q, k_cache, head_dim), "attn_decode_f32: 32-bit operands, head width and pages "
          "that are multiples of 4")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= heads * head_dim, "attention: q")
    _need(out.shape == (q.shape[0], heads * head_dim) and out.is_contiguous() and out.dtype == q.dtype, "attention: out")
    _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, q.dtype), "attention: cache shape or dtype")
    count = entries.numel()
    _need(entries.dtype == torch.int32 and entries.is_contiguous(), "attention: entries")
    _need(partial.dtype == torch.float32 and partial.is_contiguous()
          and partial.numel() >= count * heads * chunks * (head_dim + 2), "attention: workspace too small")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(), "attention: table")
    _need(entry_start.dtype == torch.int32 and entry_first_pos.dtype == torch.int32
          and entry_start.numel() == block_table.shape[0] + 1 and entry_first_pos.numel() == block_table.shape[0],
          "attention: entry arrays")
    _need(heads % kv_heads == 0 and chunks >= 1, "attention: heads must be a multiple of kv_heads")
    fn = _fn("attn_generic", "vk_attn_decode_f32_ext",
             [_p, _ll, _p, _p, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _f, _i, _p, _p, _i, _i, _p])
    _status(fn(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(partial), _ptr(entries), count,
               _ptr(entry_start), _ptr(entry_first_pos), _ptr(block_table), block_table.shape[1], k_cache.shape[2],
               heads, kv_heads, head_dim, float(scale), int(window), float(softcap), int(chunks),
               *attn_extras_args(extras, heads, window), _stream()), "attn_decode_f32")


ATTN_PREFILL_F32_MAX_HEAD_DIM = 128   # the K, V and weight tiles of a wider head do not fit a CU's LDS


def attn_prefill_f32_supported(q: torch.Tensor, k_cache: torch.Tensor, head_dim: int) -> bool:
    """Whether :func:`attn_prefill_f32` takes the operands: all 32-bit, a head width that is a multiple of 16 and
    at most 128, pages of a multiple of 4 positions, 16-byte rows."""
    return (q.dtype == torch.float32 and k_cache.dtype == torch.float32 and head_dim % 16 == 0
            and head_dim <= ATTN_PREFILL_F32_MAX_HEAD_DIM and k_cache.shape[2] % 4 == 0 and q.stride(0) % 4 == 0
            and q.data_ptr() % 16 == 0)


def attn_prefill_f32(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                     tiles: torch.Tensor, tile_tokens: int, entry_start: torch.Tensor, entry_first_pos: torch.Tensor,
                     block_table: torch.Tensor, heads: int, kv_heads: int, head_dim: int, scale: float,
                     window: int, softcap: float = 0.0, extras=None) -> None:
    """32-bit attention of the entries' tiles listed in ``tiles`` (pairs: entry, first token within it; ``tile_tokens``
    tokens a tile, a multiple of 64): 64 tokens of one head a workgroup, the positions in LDS tiles of 64."""
    _dev(q, k_cache, v_cache, out, tiles, entry_start, entry_first_pos, block_table)
    _need(attn_prefill_f32_supported(q, k_cache, head_dim), "attn_prefill_f32: 32-bit operands, a head width that is a "
          "multiple of 16 up to 128, pages of a multiple of 4 positions")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= heads * head_dim, "attention: q")
    _need(out.shape == (q.shape[0], heads * head_dim) and out.is_contiguous() and out.dtype == q.dtype, "attention: out")
    _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, q.dtype), "attention: cache shape or dtype")
    _need(tiles.dtype == torch.int32 and tiles.numel() % 2 == 0 and tiles.is_contiguous(), "attention: tiles")
    _need(tile_tokens >= 64 and tile_tokens % 64 == 0, "attention: tokens of a tile must be a multiple of 64")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(), "attention: table")
    _need(entry_start.dtype == torch.int32 and entry_first_pos.dtype == torch.int32
          and entry_start.numel() == block_table.shape[0] + 1 and entry_first_pos.numel() == block_table.shape[0],
          "attention: entry arrays")
    _need(heads % kv_heads == 0, "attention: heads must be a multiple of kv_heads")
    fn = _fn("attn_generic", "vk_attn_prefill_f32_ext",
             [_p, _ll, _p, _p, _p, _p, _i, _i, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _f, _p, _p, _i, _i, _p])
    _status(fn(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(tiles), tiles.numel() // 2,
               int(tile_tokens), _ptr(entry_start), _ptr(entry_first_pos), _ptr(block_table), block_table.shape[1],
               k_cache.shape[2], heads, kv_heads, head_dim, float(scale), int(window), float(softcap),
               *attn_extras_args(extras, heads, window), _stream()), "attn_prefill_f32")


# ----------------------------------------------------------------------------------------------
SAMPLE_SLICES = 32
SAMPLE_SLICES_FROM = 32_768   # columns from which a row's best logit is searched in slices


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, uniform: Optional[torch.Tensor], out: torch.Tensor,
           slot: Optional[torch.Tensor] = None, position: Optional[torch.Tensor] = None,
           reseed: Optional[torch.Tensor] = None, seed_state: Optional[torch.Tensor] = None,
           slot_table: Optional[torch.Tensor] = None) -> None:
    """One token per row: greedy where ``temperature`` is 0, else a draw after the top-k/top-p/min-p cuts.

    ``out[r]`` is -1 when row ``r`` has no finite logit.  The uniform of a row that draws is ``uniform[r]``, or
    with a ``slot_table`` (int64 ``[slots, 2]``: generator state and next position per state slot) the next
    output of the xorshift64* generator in slot ``slot[r]``, which the kernel advances; ``reseed[r]`` puts
    ``seed_state[r]`` there first, and ``position[r]`` is recorded beside it.
    """
    _dev(logits, temperature, top_k, top_p, min_p, uniform, out, slot, position, reseed, seed_state, slot_table)
    rows, vocab = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "sample: logits must be contiguous float32")
    columns = [("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
               ("top_p", top_p, torch.float32), ("min_p", min_p, torch.float32), ("out", out, torch.int32)]
    if slot_table is None:
        _need(uniform is not None, "sample: either uniforms or a table of state slots")
        columns.append(("uniform", uniform, torch.float64))
    else:
        _need(slot_table.dtype == torch.int64 and slot_table.dim() == 2 and slot_table.shape[1] == 2
              and slot_table.is_contiguous(), "sample: the slot table must be contiguous int64 [slots, 2]")
        columns += [("slot", slot, torch.int32), ("position", position, torch.int32), ("reseed", reseed, torch.int32),
                    ("seed_state", seed_state, torch.int64)]
    for name, tensor, dtype in columns:
        _need(tensor is not None and tensor.dtype == dtype and tensor.numel() == rows and tensor.is_contiguous(),
              f"sample: {name} must hold one {dtype} per row")
    # a wide vocabulary: the rows' best logits are found by 32 workgroups a row before the one that draws
    slices = SAMPLE_SLICES if vocab >= SAMPLE_SLICES_FROM else 0
    best = torch.empty(rows * slices, dtype=torch.float32, device=logits.device) if slices else None
    best_id = torch.empty(rows * slices, dtype=torch.int32, device=logits.device) if slices else None
    fn = _fn("sampling", "vk_sample", [_p, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _p, _p, _p, _p, _i, _p])
    _status(fn(_ptr(logits), rows, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(min_p), _ptr(uniform),
               _ptr(out), _ptr(best), _ptr(best_id), slices, _ptr(slot), _ptr(position), _ptr(reseed),
               _ptr(seed_state), _ptr(slot_table), slot_table.shape[0] if slot_table is not None else 0, _stream()),
            "sample")


def penalize(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor, counts: torch.Tensor,
             repetition: torch.Tensor, presence: torch.Tensor, frequency: torch.Tensor) -> None:
    """Apply the repetition, presence and frequency penalties in place to the listed (row, token) pairs."""
    _dev(logits, rows, tokens, counts, repetition, presence, frequency)
    num_rows, vocab = logits.shape
    n = rows.numel()
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "penalize: logits must be contiguous float32")
    _need(tokens.numel() == n and counts.numel() == n and all(t.dtype == torch.int32 for t in (rows, tokens, counts)),
          "penalize: rows, tokens and counts must be int32 of one length")
    _need(all(t.dtype == torch.float32 and t.numel() == num_rows for t in (repetition, presence, frequency)),
          "penalize: one float32 factor per row")
    if n:
        _need(int(rows.max()) < num_rows and int(rows.min()) >= 0, "penalize: row index out of range")
    fn = _fn("sampling", "vk_penalize", [_p, _i, _p, _p, _p, _p, _p, _p, _i, _p])
    _status(fn(_ptr(logits), vocab, _ptr(rows), _ptr(tokens), _ptr(counts), _ptr(repetition), _ptr(presence),
               _ptr(frequency), n, _stream()), "penalize")


def logit_bias(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor, values: torch.Tensor) -> None:
    """``logits[rows[i], tokens[i]] += values[i]`` (pairs are unique)."""
    _dev(logits, rows, tokens, values)
    num_rows, vocab = logits.shape
    n = rows.numel()
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "logit_bias: logits must be contiguous float32")
    _need(tokens.numel() == n and values.numel() == n and rows.dtype == torch.int32 and tokens.dtype == torch.int32
          and values.dtype == torch.float32, "logit_bias: operand types")
    if n:
        _need(int(rows.max()) < num_rows and int(rows.min()) >= 0, "logit_bias: row index out of range")
    fn = _fn("sampling", "vk_logit_bias", [_p, _i, _p, _p, _p, _i, _p])
    _status(fn(_ptr(logits), vocab, _ptr(rows), _ptr(tokens), _ptr(values), n, _stream()), "logit_bias")


# ----------------------------------------------------------------------------------------------
def gemm_bf16_supported(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
    """Whether the matrix-core kernels take these operands (16-byte chunks along K, rows short enough for their
    32-bit offsets); what they do not take goes to the 32-bit FMA kernel."""
    k = a.shape[1]
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype in _DT and k % 8 == 0
            and k < GEMM_BF16_MAX_K and a.stride(0) < GEMM_BF16_MAX_K
            and a.stride(1) == 1 and (a.stride(0) % 8 == 0 or a.shape[0] == 1) and a.data_ptr() % 16 == 0
            and w.is_contiguous() and w.data_ptr() % 16 == 0 and out.stride(1) == 1)


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
              accumulate: bool = False, skinny_limit: int = 64, skinny_shape: int = 0) -> None:
    """``out (+)= a @ w.T + bias`` on the matrix cores: bfloat16 products, 32-bit sums."""
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm: operands must be matrices")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n), f"gemm: shapes {tuple(a.shape)} x {tuple(w.shape)}^T -> {tuple(out.shape)}")
    _need(gemm_bf16_supported(a, w, out), "gemm_bf16: operands must be bfloat16, K a multiple of 8, rows 16-byte aligned")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    if accumulate:
        _need(out.dtype == torch.float32, "gemm: accumulation needs a float32 output")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n)
    _need(ldc >= n, "gemm: out's row stride")
    partial = None
    if m > skinny_limit or m > 64:  # the tiled kernel may split K into a workspace of at most eight ranges
        partial = _split_k_workspace(a.device, min(8 * m * n, _TILE_WORKSPACE_FLOATS), "tile")
    fn = _fn("gemm_bf16", "vk_gemm_bf16", [_p, _p, _p, _p, _i, _i, _i, _i, _ll, _ll, _i, _i, _i, _p, _ll, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), _dt(out, "out"), m, n, k, lda, ldc, 1 if accumulate else 0,
               int(skinny_limit), int(skinny_shape), _ptr(partial), partial.numel() if partial is not None else 0,
               _stream()), "gemm_bf16")


def gemm_bf16_qkv_rope_supported(a: torch.Tensor, w: torch.Tensor, qkv: torch.Tensor, head_dim: int) -> bool:
    """Whether :func:`gemm_bf16_qkv_rope` takes the operands: all bfloat16, at most 16 tokens, an even head
    width, a contiguous output, a weight of less than 2 GiB."""
    return (qkv.dtype == torch.bfloat16 and 1 <= a.shape[0] <= 16 and head_dim % 2 == 0 and qkv.is_contiguous()
            and gemm_bf16_supported(a, w, qkv) and w.shape[0] * w.shape[1] * 2 < 2 ** 31)


def gemm_bf16_qkv_rope(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], qkv: torch.Tensor,
                       positions: torch.Tensor, inv_freq: torch.Tensor, k_cache: Optional[torch.Tensor],
                       v_cache: Optional[torch.Tensor], entry_of_token: torch.Tensor, block_table: Optional[torch.Tensor],
                       heads: int, kv_heads: int, head_dim: int, sumsq: Optional[torch.Tensor] = None, groups: int = 0,
                       eps: float = 0.0) -> None:
    """``qkv = a @ w.T + bias`` for up to 16 tokens with the full rotation of its q and k heads and the write of
    the tokens' K and V into their pages in the product's epilogue: what :func:`gemm_bf16` followed by
    :func:`rope_kvwrite` (without a table of angles) leaves, in one launch.  With ``sumsq``, ``a`` is ``x * gain`` as
    :func:`gemm_bf16_follow` left it and the product's sums are divided by the root mean square of ``x`` (from the
    ``groups`` sums of squares and ``eps``) before the bias: the norm in front of the product costs no kernel."""
    _dev(a, w, bias, qkv, positions, inv_freq, k_cache, v_cache, entry_of_token, block_table, sumsq)
    if sumsq is not None:
        _need(sumsq.dtype == torch.float32 and 1 <= groups <= 512 and sumsq.numel() >= groups * 16,
              "gemm_bf16_qkv_rope: sumsq")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and qkv.shape == (m, n) and n == (heads + 2 * kv_heads) * head_dim, "gemm_bf16_qkv_rope: shapes")
    _need(gemm_bf16_qkv_rope_supported(a, w, qkv, head_dim), "gemm_bf16_qkv_rope: bfloat16 operands, at most 16 tokens, "
          "an even head width")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    _need(positions.dtype == torch.int32 and positions.numel() >= m, "gemm_bf16_qkv_rope: positions")
    _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == head_dim // 2 and inv_freq.is_contiguous(),
          "gemm_bf16_qkv_rope: inv_freq must hold head_dim / 2 floats")
    table_width = block_size = 0
    if k_cache is not None:
        _need(v_cache is not None and block_table is not None, "gemm_bf16_qkv_rope: cache without table")
        _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, qkv.dtype), "gemm_bf16_qkv_rope: cache shape or dtype")
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
              "gemm_bf16_qkv_rope: block table")
        _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() >= m, "gemm_bf16_qkv_rope: entries")
        table_width, block_size = block_table.shape[1], k_cache.shape[2]
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    fn = _fn("gemm_bf16", "vk_gemm_bf16_qkv_rope",
             [_p, _p, _p, _p, _i, _i, _i, _ll, _ll, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _i, _f, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(qkv), m, n, k, lda, n, _ptr(positions), _ptr(inv_freq), _ptr(k_cache),
               _ptr(v_cache), _ptr(entry_of_token), _ptr(block_table), table_width, block_size, heads, kv_heads, head_dim,
               _ptr(sumsq), int(groups), float(eps), _stream()), "gemm_bf16_qkv_rope")


def gemm_bf16_follow_supported(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
    """Whether :func:`gemm_bf16_follow` takes the operands: bfloat16 product of up to 16 tokens into a float32
    residual whose width is a multiple of four and at most 8,192 (512 workgroups of 16 columns)."""
    return (out.dtype == torch.float32 and 1 <= a.shape[0] <= 16 and out.shape[1] % 4 == 0 and out.shape[1] <= 8192
            and out.is_contiguous() and gemm_bf16_supported(a, w, out))


def follow_stride(tokens: int) -> int:
    """Floats per group of the sums of squares that the first half of a split norm leaves for ``tokens`` rows: 16 for
    up to 16 tokens, else the tokens rounded up to a multiple of 64."""
    return 16 if tokens <= 16 else (tokens + 63) // 64 * 64


def follow_sumsq_floats(n: int, tokens: int) -> int:
    """Floats that the sums of squares of :func:`gemm_bf16_follow` and :func:`gemm_bf16_mid_follow` may take for an
    output of ``n`` columns and ``tokens`` rows (16 per workgroup that owns at least 8 columns, or a
    :func:`follow_stride` per 1,024 columns)."""
    return max(((n + 7) // 8) * 16, ((n + 1023) // 1024) * follow_stride(tokens))


def gemm_bf16_follow(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                     gain: torch.Tensor, scaled: torch.Tensor, sumsq: torch.Tensor) -> int:
    """``out += a @ w.T + bias`` (``out`` float32: the residual) for up to 16 tokens, and the first half of the RMS
    norm that follows: ``scaled = bfloat16(out * gain)`` and per workgroup the sums of squares of its columns
    (``sumsq[groups, 16]``).  Returns ``groups``; :func:`gemm_bf16_gated_scaled` does the other half."""
    _dev(a, w, bias, out, gain, scaled, sumsq)
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n) and scaled.shape == (m, n), "gemm_bf16_follow: shapes")
    _need(gemm_bf16_follow_supported(a, w, out), "gemm_bf16_follow: bfloat16 operands, a float32 output, at most 16 tokens")
    _need(scaled.dtype == torch.bfloat16 and scaled.is_contiguous(), "gemm_bf16_follow: scaled must be bfloat16 [m, n]")
    _need(gain.dtype == torch.float32 and gain.numel() == n and gain.is_contiguous(), "gemm_bf16_follow: gain must be float32 [n]")
    _need(sumsq.dtype == torch.float32 and sumsq.is_contiguous() and sumsq.numel() >= follow_sumsq_floats(n, m),
          "gemm_bf16_follow: sumsq is too small")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    groups = ctypes.c_int(0)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_follow", [_p, _p, _p, _p, _i, _i, _i, _ll, _ll, _p, _p, _ll, _p, _ll,
                                                  ctypes.POINTER(ctypes.c_int), _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), m, n, k, lda, n, _ptr(gain), _ptr(scaled), n, _ptr(sumsq),
               sumsq.numel(), ctypes.byref(groups), _stream()), "gemm_bf16_follow")
    return int(groups.value)


def gemm_bf16_mid_follow(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                         ranges: int, rows_per_wave: int, gain: torch.Tensor, scaled: torch.Tensor,
                         sumsq: torch.Tensor) -> int:
    """:func:`gemm_bf16_follow` for up to 64 tokens where K is split into ``ranges`` > 1 over workgroups
    (:func:`gemm_bf16_mid` with accumulation): the kernel that adds the ranges leaves ``scaled`` and the sums of
    squares, :func:`follow_stride` floats per group.  Returns the number of groups."""
    _dev(a, w, bias, out, gain, scaled, sumsq)
    m, k = a.shape
    n = w.shape[0]
    _need(m <= 64 and ranges >= 2, "gemm_bf16_mid_follow: at most 64 tokens and at least two ranges")
    _need(w.shape[1] == k and out.shape == (m, n) and scaled.shape == (m, n), "gemm_bf16_mid_follow: shapes")
    _need(out.dtype == torch.float32 and out.is_contiguous() and gemm_bf16_supported(a, w, out),
          "gemm_bf16_mid_follow: bfloat16 operands and a float32 output")
    _need(scaled.dtype == torch.bfloat16 and scaled.is_contiguous(), "gemm_bf16_mid_follow: scaled must be bfloat16 [m, n]")
    _need(gain.dtype == torch.float32 and gain.numel() == n and gain.is_contiguous(), "gemm_bf16_mid_follow: gain")
    _need(sumsq.dtype == torch.float32 and sumsq.is_contiguous() and sumsq.numel() >= follow_sumsq_floats(n, m),
          "gemm_bf16_mid_follow: sumsq is too small")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    partial = _split_k_workspace(a.device, ranges * 64 * n, "mid")
    groups = ctypes.c_int(0)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_mid_follow", [_p, _p, _p, _p, _i, _i, _i, _ll, _ll, _i, _i, _p, _ll, _p, _p, _ll, _p,
                                                      _ll, _i, ctypes.POINTER(ctypes.c_int), _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), m, n, k, lda, n, int(ranges), int(rows_per_wave), _ptr(partial),
               partial.numel(), _ptr(gain), _ptr(scaled), n, _ptr(sumsq), sumsq.numel(), follow_stride(m),
               ctypes.byref(groups), _stream()), "gemm_bf16_mid_follow")
    return int(groups.value)


def gemm_bf16_mid_qkv_rope(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], qkv: torch.Tensor,
                           ranges: int, rows_per_wave: int, positions: torch.Tensor, inv_freq: torch.Tensor,
                           k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], entry_of_token: torch.Tensor,
                           block_table: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int,
                           sumsq: Optional[torch.Tensor] = None, groups: int = 0, eps: float = 0.0) -> None:
    """:func:`gemm_bf16_qkv_rope` for up to 64 tokens where K is split into ``ranges`` > 1 over workgroups: the
    kernel that adds the ranges also divides by the norm (``sumsq``: ``groups`` groups of :func:`follow_stride`
    floats), adds the bias, rotates and writes the cache."""
    _dev(a, w, bias, qkv, positions, inv_freq, k_cache, v_cache, entry_of_token, block_table, sumsq)
    m, k = a.shape
    n = w.shape[0]
    _need(m <= 64 and ranges >= 2 and head_dim % 8 == 0, "gemm_bf16_mid_qkv_rope: at most 64 tokens, two ranges or more, "
          "a head width that is a multiple of 8")
    _need(w.shape[1] == k and qkv.shape == (m, n) and n == (heads + 2 * kv_heads) * head_dim, "gemm_bf16_mid_qkv_rope: shapes")
    _need(qkv.dtype == torch.bfloat16 and qkv.is_contiguous() and gemm_bf16_supported(a, w, qkv),
          "gemm_bf16_mid_qkv_rope: bfloat16 operands and a contiguous output")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    _need(positions.dtype == torch.int32 and positions.numel() >= m, "gemm_bf16_mid_qkv_rope: positions")
    _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == head_dim // 2 and inv_freq.is_contiguous(),
          "gemm_bf16_mid_qkv_rope: inv_freq must hold head_dim / 2 floats")
    table_width = block_size = 0
    if k_cache is not None:
        _need(v_cache is not None and block_table is not None, "gemm_bf16_mid_qkv_rope: cache without table")
        _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, qkv.dtype), "gemm_bf16_mid_qkv_rope: cache shape or dtype")
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
              "gemm_bf16_mid_qkv_rope: block table")
        _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() >= m, "gemm_bf16_mid_qkv_rope: entries")
        table_width, block_size = block_table.shape[1], k_cache.shape[2]
    if sumsq is not None:
        _need(sumsq.dtype == torch.float32 and groups >= 1 and sumsq.numel() >= groups * follow_stride(m),
              "gemm_bf16_mid_qkv_rope: sumsq")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    partial = _split_k_workspace(a.device, ranges * 64 * n, "mid")
    fn = _fn("gemm_bf16", "vk_gemm_bf16_mid_qkv_rope",
             [_p, _p, _p, _p, _i, _i, _i, _ll, _ll, _i, _i, _p, _ll, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _i, _i, _f, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(qkv), m, n, k, lda, n, int(ranges), int(rows_per_wave), _ptr(partial),
               partial.numel(), _ptr(positions), _ptr(inv_freq), _ptr(k_cache), _ptr(v_cache), _ptr(entry_of_token),
               _ptr(block_table), table_width, block_size, heads, kv_heads, head_dim, _ptr(sumsq), int(groups),
               follow_stride(m), float(eps), _stream()), "gemm_bf16_mid_qkv_rope")


def gemm_bf16_gated_scaled(scaled: torch.Tensor, w: torch.Tensor, out: torch.Tensor, sumsq: torch.Tensor, groups: int,
                           eps: float) -> None:
    """:func:`gemm_bf16_gated` with resident activations on what :func:`gemm_bf16_follow` left: ``scaled`` is
    ``x * gain`` in bfloat16, and gate and up are divided by the root mean square of ``x`` (from the ``groups``
    sums of squares and ``eps``) before the activation."""
    _dev(scaled, w, out, sumsq)
    m, k = scaled.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n // 2) and n % 32 == 0, "gemm_gated: shapes")
    _need(gemm_bf16_supported(scaled, w, out) and out.dtype == torch.bfloat16, "gemm_gated: operands must be bfloat16")
    _need(sumsq.dtype == torch.float32 and sumsq.numel() >= groups * 16 and groups >= 1, "gemm_bf16_gated_scaled: sumsq")
    lda = scaled.stride(0) if m > 1 else max(scaled.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n // 2)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_gated_scaled", [_p, _p, _p, _i, _i, _i, _ll, _ll, _p, _i, _f, _p])
    _status(fn(_ptr(scaled), _ptr(w), _ptr(out), m, n, k, lda, ldc, _ptr(sumsq), int(groups), float(eps), _stream()),
            "gemm_bf16_gated_scaled")


def gemm_bf16_gated_tile_scaled(scaled: torch.Tensor, w: torch.Tensor, out: torch.Tensor, sumsq: torch.Tensor,
                                groups: int, eps: float) -> None:
    """:func:`gemm_bf16_gated` on the tiled kernel, for any number of tokens, on the first half of a split norm:
    ``scaled`` is ``x * gain`` in bfloat16, and gate and up are divided by the root mean square of ``x`` (from the
    ``groups`` sums of squares, :func:`follow_stride` floats each, and ``eps``) before the activation."""
    _dev(scaled, w, out, sumsq)
    m, k = scaled.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n // 2) and n % 32 == 0, "gemm_gated: shapes")
    _need(gemm_bf16_supported(scaled, w, out) and out.dtype == torch.bfloat16, "gemm_gated: operands must be bfloat16")
    stride = follow_stride(m)
    _need(sumsq.dtype == torch.float32 and sumsq.is_contiguous() and groups >= 1 and sumsq.numel() >= groups * stride,
          "gemm_bf16_gated_tile_scaled: sumsq")
    lda = scaled.stride(0) if m > 1 else max(scaled.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n // 2)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_gated_tile_scaled", [_p, _p, _p, _i, _i, _i, _ll, _ll, _p, _i, _i, _f, _p])
    _status(fn(_ptr(scaled), _ptr(w), _ptr(out), m, n, k, lda, ldc, _ptr(sumsq), int(groups), stride, float(eps), _stream()),
            "gemm_bf16_gated_tile_scaled")


TILE_TILINGS = {0: "128x128 staged", 2: "256x128 staged", 3: "128x256 staged", 4: "256x256 staged",
                9: "128x128 direct", 7: "256x128 direct", 8: "128x256 direct", 5: "256x256 direct", 6: "256x192 direct",
                10: "128x96 direct, gated only", 11: "128x160 direct, gated only", 12: "128x224 direct, gated only"}


def gemm_bf16_force_tiling(tiling: int = -1, ranges: int = 1, stages: int = 0) -> None:
    """For tests and measurements: make the tiled kernel of :func:`gemm_bf16` and :func:`gemm_bf16_gated`
    use one tiling (a key of ``TILE_TILINGS``) and split K into ``ranges``; ``-1`` gives the choice back
    to the launcher.  A "direct" tiling falls back to its staged twin when K is no multiple of 64.  ``stages``:
    2 or 3 LDS stages for the direct 128-token tilings (0: three up to 128 tokens, else two)."""
    if tiling >= 0:
        _need(tiling in TILE_TILINGS and 1 <= ranges <= 8, "gemm_bf16_force_tiling: unknown tiling or ranges")
    _need(stages in (0, 2, 3), "gemm_bf16_force_tiling: stages are 0 (by shape), 2 or 3")
    fn = _fn("gemm_bf16", "vk_gemm_bf16_tile_config", [_i, _i, _i])
    _status(fn(-1 if tiling < 0 else tiling, int(ranges), int(stages)), "gemm_bf16_force_tiling")


def gemm_bf16_force_tile_group(rows: int = 0) -> None:
    """For measurements: the tiled kernel walks its tiles in blocks of ``rows`` rows of tiles (0: chosen by shape)."""
    fn = _fn("gemm_bf16", "vk_gemm_bf16_tile_group", [_i])
    _status(fn(int(rows)), "gemm_bf16_force_tile_group")


# ----------------------------------------------------------------------------------------------
def attn_bf16_padded_width(head_dim: int) -> int:
    """The padded head width a matrix-core attention module is compiled for (a multiple of 32)."""
    return (head_dim + 31) // 32 * 32


def attn_bf16_supported(q: torch.Tensor, k_cache: torch.Tensor, head_dim: int) -> bool:
    return (q.dtype == torch.bfloat16 and head_dim % 8 == 0 and head_dim <= 256 and k_cache.shape[2] % 8 == 0
            and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0)


def attn_bf16_prefill_loads_directly(k_cache: torch.Tensor, kv_heads: int, head_dim: int) -> bool:
    """Whether prompt attention runs on the kernel that loads K and V tiles straight into LDS (which alone can cut a
    tile's positions into chunks): a head width of 64, 128 or 256 and pages of 8, 16, 32 or 64 positions."""
    block_size = k_cache.shape[2]
    return (head_dim in (64, 128, 256) and block_size in (8, 16, 32, 64)
            and kv_heads * block_size * head_dim * 2 < 2 ** 32)


ATTN_PREFILL_PARTIAL_ROW_EXTRA = 4   # floats beside the padded head width in a column's partial result


def attn_bf16_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                      tiles: torch.Tensor, entry_start: torch.Tensor, entry_first_pos: torch.Tensor,
                      block_table: torch.Tensor, heads: int, kv_heads: int, head_dim: int, scale: float,
                      window: int, split: bool = False, chunk_tiles: int = 0, max_chunks: int = 0,
                      softcap: float = 0.0, extras=None) -> None:
    """Attention of the entries' 128-token tiles listed in ``tiles`` (pairs: entry, first token within it).
    ``split``: workgroups of sixteen waves that halve a tile's positions between them and merge at the end, where
    the kernel in use has that form (for few tiles of very different lengths); the same result up to rounding.
    ``chunk_tiles`` > 0 (where :func:`attn_bf16_prefill_loads_directly`): a tile's steps of 64 positions are cut into
    chunks of that many, a workgroup each, and a second kernel merges them; no tile may have more than ``max_chunks``."""
    _dev(q, k_cache, v_cache, out, tiles, entry_start, entry_first_pos, block_table)
    _need(attn_bf16_supported(q, k_cache, head_dim), "attn_bf16: operands must be bfloat16 with 16-byte rows")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= heads * head_dim, "attention: q")
    _need(out.shape == (q.shape[0], heads * head_dim) and out.is_contiguous() and out.dtype == q.dtype, "attention: out")
    _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, q.dtype), "attention: cache shape or dtype")
    _need(tiles.dtype == torch.int32 and tiles.numel() % 2 == 0 and tiles.is_contiguous(), "attention: tiles")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(), "attention: table")
    _need(entry_start.dtype == torch.int32 and entry_first_pos.dtype == torch.int32
          and entry_start.numel() == block_table.shape[0] + 1 and entry_first_pos.numel() == block_table.shape[0],
          "attention: entry arrays")
    num_tiles = tiles.numel() // 2
    partial = None
    if chunk_tiles > 0 and attn_bf16_prefill_loads_directly(k_cache, kv_heads, head_dim):
        _need(max_chunks >= 1, "attention: max_chunks")
        partial = torch.empty(num_tiles * heads * max_chunks * 128 * (head_dim + ATTN_PREFILL_PARTIAL_ROW_EXTRA),
                              dtype=torch.float32, device=q.device)
    else:
        chunk_tiles = max_chunks = 0
    module = f"attn_bf16_hd{attn_bf16_padded_width(head_dim)}"
    fn = _fn(module, "vk_attn_bf16_prefill_ext",
             [_p, _ll, _p, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _f, _i, _p, _ll, _i, _i, _p, _p, _i, _i, _p],
             key=module + ".prefill")
    _status(fn(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(tiles), num_tiles,
               _ptr(entry_start), _ptr(entry_first_pos), _ptr(block_table), block_table.shape[1], k_cache.shape[2],
               heads, kv_heads, head_dim, float(scale), int(window), float(softcap), 1 if split else 0, _ptr(partial),
               partial.numel() if partial is not None else 0, int(chunk_tiles), int(max_chunks),
               *attn_extras_args(extras, heads, window), _stream()),
            "attn_bf16_prefill")


ATTN_DECODE_JOINED_CHUNKS = 8   # waves of a workgroup that merges its chunks itself


def attn_bf16_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                     partial: torch.Tensor, entries: torch.Tensor, entry_start: torch.Tensor,
                     entry_first_pos: torch.Tensor, block_table: torch.Tensor, heads: int, kv_heads: int,
                     head_dim: int, scale: float, window: int, chunk: int, chunks: int, dense: bool = False,
                     join: bool = False, softcap: float = 0.0, extras=None) -> None:
    """Attention of the single-token entries listed in ``entries``, positions split into ``chunks`` of ``chunk``.
    ``dense``: the step holds single-token entries only, so entry i is the i-th of them and holds token i; the
    kernel then need not look either up.  ``join``: one workgroup per entry and key head takes all chunks (at most
    ``ATTN_DECODE_JOINED_CHUNKS``), a wave each, and merges them itself; ``partial`` is then not used and may be
    None."""
    _dev(q, k_cache, v_cache, out, partial, entries, entry_start, entry_first_pos, block_table)
    _need(attn_bf16_supported(q, k_cache, head_dim), "attn_bf16: operands must be bfloat16 with 16-byte rows")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= heads * head_dim, "attention: q")
    _need(out.shape == (q.shape[0], heads * head_dim) and out.is_contiguous() and out.dtype == q.dtype, "attention: out")
    _need(_cache_ok(k_cache, v_cache, kv_heads, head_dim, q.dtype), "attention: cache shape or dtype")
    count = entries.numel()
    _need(entries.dtype == torch.int32 and entries.is_contiguous(), "attention: entries")
    if join:
        _need(chunks <= ATTN_DECODE_JOINED_CHUNKS, "attention: too many chunks for one workgroup")
    else:
        _need(partial is not None and partial.dtype == torch.float32 and partial.is_contiguous()
              and partial.numel() >= count * heads * chunks * (head_dim + 2), "attention: workspace too small")
    _need(chunk >= 32 and chunk % 32 == 0 and chunks >= 1, "attention: chunk must be a multiple of 32")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(), "attention: table")
    module = f"attn_bf16_hd{attn_bf16_padded_width(head_dim)}"
    fn = _fn(module, "vk_attn_bf16_decode_ext",
             [_p, _ll, _p, _p, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _f, _i, _f, _i, _i, _i, _i, _p, _p, _i, _i, _p],
             key=module + ".decode")
    _status(fn(_ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(out), _ptr(partial), _ptr(entries), count,
               _ptr(entry_start), _ptr(entry_first_pos), _ptr(block_table), block_table.shape[1], k_cache.shape[2],
               heads, kv_heads, head_dim, float(scale), int(window), float(softcap), int(chunk), int(chunks), 1 if dense else 0,
               1 if join else 0, *attn_extras_args(extras, heads, window), _stream()),
            "attn_bf16_decode")


_workspaces = {}
_retired = []  # outgrown workspaces: kept alive, since a captured graph may still write to them
_TILE_WORKSPACE_FLOATS = 64 * 1024 * 1024   # 256 MB: the most the tiled kernel's K ranges may take


def _split_k_workspace(device: torch.device, floats: int, kind: str) -> torch.Tensor:
    """Partial-sum workspace of a device and a kind of product; grown when a product needs more, never shrunk.

    Every product of the kind on the device shares it, which is safe because products run on one stream.
    """
    key = (device, kind)
    entry = _workspaces.get(key)
    if entry is None or entry.numel() < floats:
        if entry is not None:
            _retired.append(entry)
        entry = torch.empty(floats, dtype=torch.float32, device=device)
        _workspaces[key] = entry
    return entry


def gemm_bf16_mid(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                  accumulate: bool = False, ranges: int = 1, rows_per_wave: int = 2) -> None:
    """``out (+)= a @ w.T + bias`` for at most 128 rows of ``a``: activations shared through LDS, weights
    streamed; ``ranges`` > 1 splits K over workgroups and adds the ranges' partial sums in a second kernel."""
    _dev(a, w, bias, out)
    _need(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm: operands must be matrices")
    m, k = a.shape
    n = w.shape[0]
    _need(m <= 128, "gemm_bf16_mid takes at most 128 rows")
    _need(w.shape[1] == k and out.shape == (m, n), f"gemm: shapes {tuple(a.shape)} x {tuple(w.shape)}^T -> {tuple(out.shape)}")
    _need(gemm_bf16_supported(a, w, out), "gemm_bf16: operands must be bfloat16, K a multiple of 8, rows 16-byte aligned")
    _need((rows_per_wave in (1, 2) or 108 <= rows_per_wave <= 116) and ranges >= 1,
          "gemm_bf16_mid: rows_per_wave is 1 or 2 (or 108 to 116: one tile with 8 to 16 rows), ranges at least 1")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == n and bias.is_contiguous(), "gemm: bias must be float32 [n]")
    if accumulate:
        _need(out.dtype == torch.float32, "gemm: accumulation needs a float32 output")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n)
    _need(ldc >= n, "gemm: out's row stride")
    partial = None
    if ranges > 1:
        partial = _split_k_workspace(a.device, ranges * (64 if m <= 64 else 128) * n, "mid")
    fn = _fn("gemm_bf16", "vk_gemm_bf16_mid", [_p, _p, _p, _p, _i, _i, _i, _i, _ll, _ll, _i, _i, _i, _p, _ll, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), _dt(out, "out"), m, n, k, lda, ldc, 1 if accumulate else 0,
               int(ranges), int(rows_per_wave), _ptr(partial), partial.numel() if partial is not None else 0, _stream()),
            "gemm_bf16_mid")


_COMPUTE_UNITS: dict = {}


def compute_units(device: torch.device) -> int:
    """CUs of the device (cached; what the launchers with one workgroup per CU use as their grid)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _COMPUTE_UNITS:
        _COMPUTE_UNITS[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return _COMPUTE_UNITS[index]


def gemm_bf16_gated_act(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, kind: str) -> None:
    """``out = up * act(gate)`` on the tiled kernel for any number of tokens, where ``[gate, up] = a @ w.T`` and ``w``
    interleaves gate and up rows in groups of 16; ``kind``: "silu" or "gelu_tanh"."""
    _dev(a, w, out)
    m, k = a.shape
    n = w.shape[0]
    _need(kind in ("silu", "gelu_tanh"), f"gemm_gated: activation {kind!r}")
    _need(w.shape[1] == k and out.shape == (m, n // 2) and n % 32 == 0, "gemm_gated: shapes")
    _need(gemm_bf16_supported(a, w, out) and out.dtype == torch.bfloat16, "gemm_gated: operands must be bfloat16")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n // 2)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_gated_act", [_p, _p, _p, _i, _i, _i, _ll, _ll, _i, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(out), m, n, k, lda, ldc, ACTIVATIONS[kind], _stream()), "gemm_bf16_gated_act")


def gemm_bf16_gated(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, rows_per_wave: int = 1) -> None:
    """``out = up * silu(gate)`` where ``[gate, up] = a @ w.T`` and ``w`` interleaves gate and up rows in
    groups of 16.  ``out``: ``[tokens, w.shape[0] / 2]`` bfloat16.  ``rows_per_wave`` (up to 64 tokens): 1 or
    2 tiles per wave of the LDS-shared kernel, 0 for the kernel with resident activations (up to 16
    tokens, K a multiple of 128, ``tokens x K`` within LDS; refused otherwise), 3 for the tiled kernel that
    more than 64 tokens always take."""
    _dev(a, w, out)
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k and out.shape == (m, n // 2) and n % 32 == 0, "gemm_gated: shapes")
    _need(gemm_bf16_supported(a, w, out) and out.dtype == torch.bfloat16, "gemm_gated: operands must be bfloat16")
    lda = a.stride(0) if m > 1 else max(a.stride(0), k)
    lda = lda if lda % 8 == 0 else k
    ldc = out.stride(0) if m > 1 else max(out.stride(0), n // 2)
    fn = _fn("gemm_bf16", "vk_gemm_bf16_gated", [_p, _p, _p, _i, _i, _i, _ll, _ll, _i, _p])
    _status(fn(_ptr(a), _ptr(w), _ptr(out), m, n, k, lda, ldc, int(rows_per_wave), _stream()), "gemm_bf16_gated")


# ----------------------------------------------------------------------------------------------
def _f32(tensor: torch.Tensor, what: str) -> None:
    _need(tensor.dtype == torch.float32 and tensor.is_contiguous(), f"{what} must be contiguous float32")


def _i32(*tensors: torch.Tensor) -> None:
    for tensor in tensors:
        _need(tensor.dtype == torch.int32 and tensor.is_contiguous(), "index tensors must be contiguous int32")


def dyt(x: torch.Tensor, alpha: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, out: torch.Tensor,
        rows: Optional[torch.Tensor] = None) -> None:
    """``out = tanh(alpha * x) * weight + bias`` per element; ``x`` 32-bit ``[tokens, width]``, ``alpha`` one number
    on the device; ``rows`` (int32) selects rows of ``x``."""
    _dev(x, alpha, weight, bias, out, rows)
    width = x.shape[1]
    _need(x.dim() == 2 and x.dtype == torch.float32 and x.is_contiguous(), "dyt: x must be contiguous float32 [tokens, width]")
    _need(alpha.dtype == torch.float32 and alpha.numel() == 1, "dyt: alpha must be one float32")
    for name, t in (("weight", weight), ("bias", bias)):
        _need(t.dtype == torch.float32 and t.numel() == width and t.is_contiguous(), f"dyt: {name} must be float32 [width]")
    count = x.shape[0] if rows is None else rows.numel()
    if rows is not None:
        _i32(rows)
    _need(out.shape == (count, width) and out.is_contiguous(), "dyt: out shape")
    fn = _fn("elementwise", "vk_dyt", [_p, _p, _p, _p, _p, _p, _i, _i, _i, _p])
    _status(fn(_ptr(x), _ptr(alpha), _ptr(weight), _ptr(bias), _ptr(rows), _ptr(out), _dt(out, "out"), count, width,
               _stream()), "dyt")


def dyt_pair(x: torch.Tensor, first, second, out1: torch.Tensor, out2: torch.Tensor) -> None:
    """Two Dynamic Tanh norms of the same rows in one launch: ``out_k = tanh(alpha_k * x) * weight_k + bias_k``; ``first``
    and ``second`` are ``(alpha, weight, bias)`` as :func:`dyt` takes them."""
    width = x.shape[1]
    _need(x.dim() == 2 and x.dtype == torch.float32 and x.is_contiguous(), "dyt_pair: x must be contiguous float32 [tokens, width]")
    for alpha, weight, bias in (first, second):
        _dev(x, alpha, weight, bias)
        _need(alpha.dtype == torch.float32 and alpha.numel() == 1, "dyt_pair: alpha must be one float32")
        for name, t in (("weight", weight), ("bias", bias)):
            _need(t.dtype == torch.float32 and t.numel() == width and t.is_contiguous(), f"dyt_pair: {name} must be float32 [width]")
    _dev(out1, out2)
    _need(out1.shape == x.shape and out2.shape == x.shape and out1.is_contiguous() and out2.is_contiguous()
          and out1.dtype == out2.dtype, "dyt_pair: outputs")
    fn = _fn("elementwise", "vk_dyt_pair", [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _p])
    _status(fn(_ptr(x), _ptr(first[0]), _ptr(first[1]), _ptr(first[2]), _ptr(out1), _ptr(second[0]), _ptr(second[1]),
               _ptr(second[2]), _ptr(out2), _dt(out1, "out"), x.shape[0], width, _stream()), "dyt_pair")


def scale_(x: torch.Tensor, factor: float) -> None:
    """``x *= factor`` (32-bit, in place)."""
    _dev(x)
    _f32(x, "scale: x")
    fn = _fn("elementwise", "vk_scale", [_p, _f, _ll, _p])
    _status(fn(_ptr(x), float(factor), x.numel(), _stream()), "scale")


def decay_(x: torch.Tensor, w0: torch.Tensor) -> None:
    """``x = exp(-exp(x + w0))`` in place; ``x`` 32-bit ``[tokens, width]``, ``w0`` ``[width]``."""
    _dev(x, w0)
    _f32(x, "decay: x")
    _need(x.dim() == 2 and w0.dtype == torch.float32 and w0.is_contiguous() and w0.numel() == x.shape[1], "decay: w0")
    fn = _fn("recurrent", "vk_decay", [_p, _p, _i, _ll, _p])
    _status(fn(_ptr(x), _ptr(w0), x.shape[1], x.numel(), _stream()), "decay")


def tanh(x: torch.Tensor, out: torch.Tensor) -> None:
    """``out = tanh(x)``; ``x`` 32-bit, ``out`` of either dtype."""
    _dev(x, out)
    _f32(x, "tanh: x")
    _need(out.numel() == x.numel() and out.is_contiguous(), "tanh: out")
    fn = _fn("recurrent", "vk_tanh", [_p, _p, _i, _ll, _p])
    _status(fn(_ptr(x), _ptr(out), _dt(out, "out"), x.numel(), _stream()), "tanh")


# --- recurrent mixers ---------------------------------------------------------------------------
RECURRENT_MAX_KEY_DIM = 256    # a lane keeps a quarter of a state column's rows in registers: at most 64


def recurrent_head_floats(dim: int, vdim: int) -> int:
    """Floats of one head's ``[dim, vdim]`` state as the recurrence kernels keep it in a slot: padded to value tiles of
    16 and to 16, 32, 64, 128 or 256 key channels, in the order of the kernel's threads."""
    rows = 1 if dim <= 16 else 2 if dim <= 32 else 4 if dim <= 64 else 8 if dim <= 128 else 16
    return (vdim + 15) // 16 * 256 * rows


def _entries_ok(batch_arrays, num_entries: int) -> None:
    entry_start, entry_first, slots = batch_arrays
    _i32(entry_start, entry_first, slots)
    _need(entry_start.numel() >= num_entries + 1 and entry_first.numel() >= num_entries and slots.numel() >= num_entries,
          "recurrent: entry arrays are shorter than the number of entries")


def delta_prepare(proj: torch.Tensor, conv: torch.Tensor, state: torch.Tensor, conv_offset: int, entry_of: torch.Tensor,
                  entry_start: torch.Tensor, entry_first: torch.Tensor, slots: torch.Tensor, a_log: Optional[torch.Tensor],
                  dt_bias: Optional[torch.Tensor], kv_heads: int, dim: int, heads: int, vdim: int, b_col: int, a_col: int,
                  unit_eps: float, qkv: torch.Tensor, beta: torch.Tensor, decay: Optional[torch.Tensor],
                  num_entries: int) -> None:
    """Short causal convolution, silu, unit norms of q and k, beta and the decay for every token of the step (see
    ``recurrent.hip``); then the convolution's state rows are replaced by the entries' last inputs.  ``qkv`` may be the
    first columns of wider rows.  ``a_col`` below 0: no decay per head is computed (``a_log``, ``dt_bias`` and ``decay``
    may be None): the caller has one per key channel, see :func:`channel_decay`."""
    _dev(proj, conv, state, entry_of, entry_start, entry_first, slots, a_log, dt_bias, qkv, beta, decay)
    tokens = proj.shape[0]
    channels = 2 * kv_heads * dim + heads * vdim
    taps = conv.shape[1]
    _need(proj.dim() == 2 and proj.dtype == torch.float32 and proj.stride(1) == 1, "delta_prepare: proj")
    _need(proj.shape[1] >= max(channels, b_col + heads, a_col + heads) and b_col >= 0, "delta_prepare: columns")
    _need(conv.shape == (channels, taps) and taps >= 1, "delta_prepare: conv shape")
    _f32(conv, "delta_prepare: conv")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous()
          and conv_offset + (taps - 1) * channels <= state.shape[1], "delta_prepare: state row")
    _i32(entry_of)
    _need(entry_of.numel() >= tokens, "delta_prepare: entry_of")
    _entries_ok((entry_start, entry_first, slots), num_entries)
    _need(qkv.dim() == 2 and qkv.shape == (tokens, channels) and qkv.dtype == torch.float32 and qkv.stride(1) == 1
          and qkv.stride(0) >= channels, "delta_prepare: qkv")
    _need(beta.shape == (tokens, heads), "delta_prepare: beta")
    _f32(beta, "delta_prepare: beta")
    if a_col >= 0:
        for name, t in (("a_log", a_log), ("dt_bias", dt_bias)):
            _need(t is not None and t.dtype == torch.float32 and t.numel() == heads, f"delta_prepare: {name}")
        _need(decay is not None and decay.shape == (tokens, heads), "delta_prepare: decay")
        _f32(decay, "delta_prepare: decay")
    fn = _fn("recurrent", "vk_delta_prepare_strided",
             [_p, _ll, _p, _i, _p, _ll, _ll, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _f, _p, _ll, _p, _p, _i, _i, _p])
    _status(fn(_ptr(proj), proj.stride(0), _ptr(conv), taps, _ptr(state), state.stride(0), conv_offset, _ptr(entry_of),
               _ptr(entry_start), _ptr(entry_first), _ptr(slots), _ptr(a_log), _ptr(dt_bias), kv_heads, dim, heads, vdim,
               b_col, a_col, float(unit_eps), _ptr(qkv), qkv.stride(0), _ptr(beta), _ptr(decay), tokens, num_entries,
               _stream()), "delta_prepare")


def channel_decay(raw: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor, heads: int, dim: int,
                  out: torch.Tensor) -> None:
    """``out[t, h, d] = exp(-exp(a_log[h]) * softplus(raw[t, h, d] + dt_bias[h, d]))``: one decay per head and key
    channel; ``raw`` and ``out`` 32-bit ``[tokens, heads * dim]``, row-strided views are fine."""
    _dev(raw, a_log, dt_bias, out)
    tokens = raw.shape[0]
    for name, t in (("raw", raw), ("out", out)):
        _need(t.dtype == torch.float32 and t.shape == (tokens, heads * dim) and t.stride(1) == 1, f"channel_decay: {name}")
    _need(a_log.dtype == torch.float32 and a_log.numel() == heads and a_log.is_contiguous(), "channel_decay: a_log")
    _need(dt_bias.dtype == torch.float32 and dt_bias.numel() == heads * dim and dt_bias.is_contiguous(),
          "channel_decay: dt_bias")
    fn = _fn("recurrent", "vk_channel_decay", [_p, _ll, _p, _p, _i, _i, _i, _p, _ll, _p])
    _status(fn(_ptr(raw), raw.stride(0), _ptr(a_log), _ptr(dt_bias), heads, dim, tokens, _ptr(out), out.stride(0),
               _stream()), "channel_decay")


def delta_rule(qkv: torch.Tensor, beta: torch.Tensor, decay: Optional[torch.Tensor], state: torch.Tensor,
               entry_start: torch.Tensor, entry_first: torch.Tensor, slots: torch.Tensor, kv_heads: int, dim: int,
               heads: int, vdim: int, out: torch.Tensor, num_entries: int, short_entries: bool = False,
               channel_decay_col: int = -1) -> None:
    """The gated delta rule over every entry's tokens in order (``short_entries``: a step of single tokens, which
    takes the kernel's form with few registers; the result is the same), from and into the entries' state rows (the first
    ``heads * recurrent_head_floats(dim, vdim)`` floats of a row, in the kernel's own order); ``out`` 32-bit ``[tokens, heads * vdim]``.
    ``decay`` is ``[tokens, heads]``; with ``channel_decay_col`` at or above 0 there is one decay per head and key
    channel instead, ``[heads, dim]`` in every row of ``qkv`` from that column on (``qkv`` is then a view of the first
    columns of those wider rows, and ``decay`` is None)."""
    _dev(qkv, beta, decay, state, entry_start, entry_first, slots, out)
    tokens = qkv.shape[0]
    channels = 2 * kv_heads * dim + heads * vdim
    _need(qkv.shape == (tokens, channels) and qkv.dtype == torch.float32 and qkv.stride(1) == 1
          and beta.shape == (tokens, heads) and out.shape == (tokens, heads * vdim), "delta_rule: shapes")
    for t in (beta, out):
        _f32(t, "delta_rule: operands")
    if channel_decay_col >= 0:
        _need(decay is None and channel_decay_col >= channels and channel_decay_col + heads * dim <= qkv.stride(0),
              "delta_rule: the decays per channel lie behind q, k and v inside the rows of qkv")
    else:
        _need(decay is not None and decay.shape == (tokens, heads) and qkv.stride(0) == channels, "delta_rule: decay")
        _f32(decay, "delta_rule: decay")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous()
          and state.shape[1] >= heads * recurrent_head_floats(dim, vdim), "delta_rule: state row")
    _entries_ok((entry_start, entry_first, slots), num_entries)
    if dim > RECURRENT_MAX_KEY_DIM:
        raise UnsupportedError(f"delta_rule: a key width of {dim} is above the kernel's limit of {RECURRENT_MAX_KEY_DIM}")
    fn = _fn("recurrent", "vk_delta_rule_strided", [_p, _ll, _i, _p, _p, _p, _ll, _p, _p, _p, _i, _i, _i, _i, _p, _i, _i, _p])
    _status(fn(_ptr(qkv), qkv.stride(0), int(channel_decay_col), _ptr(beta), _ptr(decay), _ptr(state), state.stride(0),
               _ptr(entry_start), _ptr(entry_first), _ptr(slots), kv_heads, dim, heads, vdim, _ptr(out), num_entries,
               1 if short_entries else 0, _stream()), "delta_rule")


def memory_state_floats(heads: int, dim: int, vdim: int) -> int:
    """Floats of one request's matrix-memory state (:func:`memory_rule`): the heads' matrices, then the normalizer
    vector and the running maximum once per tile of eight value channels."""
    rows = 1 if dim <= 16 else 2 if dim <= 32 else 4 if dim <= 64 else 8 if dim <= 128 else 16
    tiles = (vdim + 15) // 16 * 2
    return heads * (recurrent_head_floats(dim, vdim) + tiles * 16 * rows + tiles)


def memory_rule(proj: torch.Tensor, q_col: int, k_col: int, v_col: int, i_col: int, f_col: int, q_scale: float, cap: float,
                state: torch.Tensor, entry_start: torch.Tensor, entry_first: torch.Tensor, slots: torch.Tensor, dim: int,
                heads: int, vdim: int, out: torch.Tensor, num_entries: int, short_entries: bool = False) -> None:
    """The matrix memory with exponential gates over every entry's tokens in order: with ``li = cap tanh(i / cap)``,
    ``lf = logsigmoid(cap tanh(f / cap))`` and a running maximum ``m`` (0 at position 0): ``m' = max(lf + m, li)``,
    ``S = exp(lf + m - m') S + exp(li - m') k v^T``, ``n`` likewise with ``k`` alone,
    ``o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)``.  q, k (``heads * dim`` each), v (``heads * vdim``) and the raw gates
    (``heads`` each) are columns of the 32-bit ``proj`` from the given offsets on; q is multiplied by ``q_scale``.  State
    rows hold :func:`memory_state_floats` floats; ``out`` 32-bit ``[tokens, heads * vdim]``.  Unless ``short_entries``
    (every entry is one token), the two gates' columns of ``proj`` are overwritten with ``li`` and ``lf``."""
    _dev(proj, state, entry_start, entry_first, slots, out)
    tokens = proj.shape[0]
    _need(proj.dim() == 2 and proj.dtype == torch.float32 and proj.stride(1) == 1, "memory_rule: proj")
    _need(min(q_col, k_col, v_col, i_col, f_col) >= 0
          and max(q_col + heads * dim, k_col + heads * dim, v_col + heads * vdim, i_col + heads, f_col + heads) <= proj.shape[1],
          "memory_rule: columns")
    _need(out.shape == (tokens, heads * vdim), "memory_rule: out shape")
    _f32(out, "memory_rule: out")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous()
          and state.shape[1] >= memory_state_floats(heads, dim, vdim), "memory_rule: state row")
    _entries_ok((entry_start, entry_first, slots), num_entries)
    _need(cap > 0.0, "memory_rule: the gates' cap must be above 0")
    if dim > RECURRENT_MAX_KEY_DIM:
        raise UnsupportedError(f"memory_rule: a key width of {dim} is above the kernel's limit of {RECURRENT_MAX_KEY_DIM}")
    fn = _fn("recurrent", "vk_memory_rule", [_p, _ll, _i, _i, _i, _i, _i, _i, _f, _f, _p, _ll, _p, _p, _p, _i, _i, _i, _p, _i, _i, _p])
    _status(fn(_ptr(proj), proj.stride(0), tokens, q_col, k_col, v_col, i_col, f_col, float(q_scale), float(cap), _ptr(state),
               state.stride(0), _ptr(entry_start), _ptr(entry_first), _ptr(slots), dim, heads, vdim, _ptr(out),
               num_entries, 1 if short_entries else 0, _stream()), "memory_rule")


def wkv_rule(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, wraw: torch.Tensor, w0: torch.Tensor,
             bonus: torch.Tensor, state: torch.Tensor, entry_start: torch.Tensor, entry_first: torch.Tensor,
             slots: torch.Tensor, dim: int, heads: int, out: torch.Tensor, num_entries: int,
             short_entries: bool = False, decayed: bool = False) -> None:
    """RWKV-style time mixing over every entry's tokens in order: ``o = (S + diag(u) k v^T)^T r``, then
    ``S = diag(w) S + k v^T`` with ``w = exp(-exp(wraw + w0))``.  ``r, k, v, wraw``: 32-bit ``[tokens, heads * dim]``
    (row-strided views are fine); state rows start with the heads' matrices
    (``heads * recurrent_head_floats(dim, dim)`` floats, in the kernel's own order).  ``decayed``: ``wraw`` already
    holds ``w`` (see :func:`decay_`)."""
    _dev(r, k, v, wraw, w0, bonus, state, entry_start, entry_first, slots, out)
    tokens, width = out.shape[0], heads * dim
    for name, t in (("r", r), ("k", k), ("v", v), ("wraw", wraw)):
        _need(t.dtype == torch.float32 and t.shape == (tokens, width) and t.stride(1) == 1, f"wkv_rule: {name}")
    for name, t in (("w0", w0), ("bonus", bonus)):
        _need(t.dtype == torch.float32 and t.numel() == width and t.is_contiguous(), f"wkv_rule: {name}")
    _f32(out, "wkv_rule: out")
    _need(out.shape == (tokens, width), "wkv_rule: out shape")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous()
          and state.shape[1] >= heads * recurrent_head_floats(dim, dim), "wkv_rule: state row")
    _entries_ok((entry_start, entry_first, slots), num_entries)
    if dim > RECURRENT_MAX_KEY_DIM:
        raise UnsupportedError(f"wkv_rule: a head width of {dim} is above the kernel's limit of {RECURRENT_MAX_KEY_DIM}")
    fn = _fn("recurrent", "vk_wkv_rule",
             [_p, _ll, _p, _ll, _p, _ll, _p, _ll, _p, _p, _p, _ll, _p, _p, _p, _i, _i, _p, _i, _i, _i, _p])
    _status(fn(_ptr(r), r.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _ptr(wraw), wraw.stride(0), _ptr(w0),
               _ptr(bonus), _ptr(state), state.stride(0), _ptr(entry_start), _ptr(entry_first), _ptr(slots), dim, heads,
               _ptr(out), num_entries, 1 if short_entries else 0, 1 if decayed else 0, _stream()), "wkv_rule")


def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, prev_offset: int, entry_of: torch.Tensor,
                entry_start: torch.Tensor, entry_first: torch.Tensor, slots: torch.Tensor, out: torch.Tensor,
                num_entries: int) -> None:
    """``out[s, t] = h[t] + (h[t - 1] - h[t]) * mu[s]``; the token before an entry's first is the state's saved row
    (``width`` floats from ``prev_offset`` on; zeros at position 0), which then takes the entry's last ``h``."""
    _dev(h, mu, state, entry_of, entry_start, entry_first, slots, out)
    tokens, width = h.shape
    mixes = mu.shape[0]
    _need(h.is_contiguous() and out.dtype == h.dtype and out.shape == (mixes, tokens, width) and out.is_contiguous(),
          "token_shift: h and out")
    _need(mu.dtype == torch.float32 and mu.shape == (mixes, width) and mu.is_contiguous(), "token_shift: mu")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous()
          and prev_offset + width <= state.shape[1], "token_shift: state row")
    _i32(entry_of)
    _need(entry_of.numel() >= tokens, "token_shift: entry_of")
    _entries_ok((entry_start, entry_first, slots), num_entries)
    fn = _fn("recurrent", "vk_token_shift", [_p, _i, _i, _p, _i, _p, _ll, _ll, _p, _p, _p, _p, _i, _i, _p, _p])
    _status(fn(_ptr(h), _dt(h, "h"), width, _ptr(mu), mixes, _ptr(state), state.stride(0), prev_offset, _ptr(entry_of),
               _ptr(entry_start), _ptr(entry_first), _ptr(slots), tokens, num_entries, _ptr(out), _stream()), "token_shift")


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, gate_silu: bool, eps: float, heads: int,
                   vdim: int, out: torch.Tensor) -> None:
    """``out[t, h] = o[t, h] / rms(o[t, h]) * weight * gate[t, h]`` per head of ``vdim`` channels; ``weight`` is
    ``[vdim]`` (shared by the heads) or ``[heads * vdim]``; ``gate`` (a row-strided view of either dtype) goes through
    silu first if ``gate_silu`` is true, or through the sigmoid if it is the string ``"sigmoid"``."""
    _dev(o, weight, gate, out)
    tokens = o.shape[0]
    _f32(o, "head_norm_gate: o")
    gate_kind = 2 if gate_silu == "sigmoid" else 1 if gate_silu in (True, "silu") else 0
    _need(o.shape == (tokens, heads * vdim) and out.shape == o.shape and out.is_contiguous(), "head_norm_gate: shapes")
    _need(weight.dtype == torch.float32 and weight.is_contiguous() and weight.numel() in (vdim, heads * vdim),
          "head_norm_gate: weight")
    _need(gate.shape == o.shape and gate.stride(1) == 1, "head_norm_gate: gate")
    fn = _fn("recurrent", "vk_head_norm_gate", [_p, _p, _i, _p, _i, _ll, _i, _f, _i, _i, _i, _p, _i, _p])
    _status(fn(_ptr(o), _ptr(weight), 1 if weight.numel() == heads * vdim and heads > 1 else 0, _ptr(gate),
               _dt(gate, "gate"), gate.stride(0), gate_kind, float(eps), heads, vdim, tokens, _ptr(out),
               _dt(out, "out"), _stream()), "head_norm_gate")


# --- latent attention -----------------------------------------------------------------------------
def latent_kv_write(x: torch.Tensor, weight: torch.Tensor, eps: float, rank: int, rot: int, rot_dims: int,
                    positions: torch.Tensor, inv_freq: Optional[torch.Tensor], entry_of: torch.Tensor,
                    table: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor) -> None:
    """A step's cached rows ``[rms_norm(x[:rank]) * weight | rotate(x[rank:rank + rot])]`` into their pages, as keys
    and transposed as values (one key head of width ``rank + rot``).  ``x``: a 32-bit row-strided view."""
    _dev(x, weight, positions, inv_freq, entry_of, table, k_cache, v_cache)
    tokens = x.shape[0]
    width = rank + rot
    _need(x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1 and x.shape[1] == width, "latent_kv_write: x")
    _need(weight.dtype == torch.float32 and weight.numel() == rank and weight.is_contiguous(), "latent_kv_write: weight")
    _need(_cache_ok(k_cache, v_cache, 1, width, k_cache.dtype), "latent_kv_write: cache shape")
    _i32(positions, entry_of, table)
    _need(positions.numel() >= tokens and entry_of.numel() >= tokens and table.dim() == 2, "latent_kv_write: indices")
    _need(rot_dims == 0 or (inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() == rot_dims // 2),
          "latent_kv_write: inv_freq")
    fn = _fn("latent", "vk_latent_kv_write", [_p, _ll, _p, _f, _i, _i, _i, _p, _p, _p, _p, _i, _i, _p, _p, _i, _i, _p])
    _status(fn(_ptr(x), x.stride(0), _ptr(weight), float(eps), rank, rot, rot_dims, _ptr(positions), _ptr(inv_freq),
               _ptr(entry_of), _ptr(table), table.shape[1], k_cache.shape[2], _ptr(k_cache), _ptr(v_cache),
               _dt(k_cache, "cache"), tokens, _stream()), "latent_kv_write")


def latent_q_rotate(q: torch.Tensor, q_head: int, q_offset: int, out: torch.Tensor, out_head: int, out_offset: int,
                    heads: int, rot: int, rot_dims: int, positions: torch.Tensor, inv_freq: Optional[torch.Tensor]) -> None:
    """``out[t, h, out_offset:out_offset + rot] = rotate(q[t, h, q_offset:q_offset + rot])`` for every head."""
    _dev(q, out, positions, inv_freq)
    tokens = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= heads * q_head and q_offset + rot <= q_head, "latent_q_rotate: q")
    _need(out.dtype == q.dtype and out.is_contiguous() and out.shape == (tokens, heads * out_head)
          and out_offset + rot <= out_head, "latent_q_rotate: out")
    _i32(positions)
    _need(rot_dims == 0 or (inv_freq is not None and inv_freq.dtype == torch.float32 and inv_freq.numel() == rot_dims // 2),
          "latent_q_rotate: inv_freq")
    fn = _fn("latent", "vk_latent_q_rotate", [_p, _ll, _i, _i, _p, _i, _i, _i, _i, _i, _p, _p, _i, _i, _p])
    _status(fn(_ptr(q), q.stride(0), q_head, q_offset, _ptr(out), out_head, out_offset, heads, rot, rot_dims,
               _ptr(positions), _ptr(inv_freq), _dt(q, "q"), tokens, _stream()), "latent_q_rotate")


def head_linear(a: torch.Tensor, a_head_stride: int, k: int, w: torch.Tensor, out: torch.Tensor,
                out_head_stride: int) -> None:
    """A product per head: ``out[t, h*so : h*so + N] = w[h] @ a[t, h*sa : h*sa + K]``; ``w``: ``[heads, N, K]``."""
    _dev(a, w, out)
    heads, n, kw = w.shape
    tokens = a.shape[0]
    _need(kw == k and w.is_contiguous(), "head_linear: w")
    _need(a.dim() == 2 and a.stride(1) == 1 and (heads - 1) * a_head_stride + k <= a.shape[1], "head_linear: a")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[0] == tokens
          and (heads - 1) * out_head_stride + n <= out.shape[1], "head_linear: out")
    fn = _fn("latent", "vk_head_linear", [_p, _i, _ll, _ll, _p, _i, _p, _i, _ll, _ll, _i, _i, _i, _i, _p])
    _status(fn(_ptr(a), _dt(a, "a"), a.stride(0), a_head_stride, _ptr(w), _dt(w, "w"), _ptr(out), _dt(out, "out"),
               out.stride(0), out_head_stride, tokens, n, k, heads, _stream()), "head_linear")


# --- mixture of experts ---------------------------------------------------------------------------
def moe_tile_rows(h: torch.Tensor, width: int, ff: int) -> int:
    """Places per tile of the experts' products for activations ``h``: 128 on the matrix cores (bfloat16, widths that
    are multiples of 8), 64 as 32-bit FMAs.  The grouping has to be made for the same number."""
    return 128 if (h.dtype == torch.bfloat16 and width % 8 == 0 and ff % 8 == 0 and h.stride(0) % 8 == 0) else 64


def moe_max_tiles(pairs: int, experts: int, tile_rows: int = 64) -> int:
    return (pairs + tile_rows - 1) // tile_rows + experts


def moe_route(logits: torch.Tensor, top: int, ids: torch.Tensor, weights: torch.Tensor, offsets: torch.Tensor,
              order: torch.Tensor, tiles: torch.Tensor, num_tiles: torch.Tensor, tile_rows: int = 64,
              groups: int = 1, keep: int = 1, all_scores=False, correction: Optional[torch.Tensor] = None,
              weight_scale: float = 1.0) -> None:
    """Each token's ``top`` largest router logits (lowest id first among equals) with the softmax over those, and the
    (token, choice) pairs grouped by expert: ``offsets [E + 1]``, ``order [T * top]``, ``tiles [max, 2]``.
    ``groups`` > 1: the experts form that many equal groups of neighbours and only those of the ``keep`` groups with
    the largest logits can be chosen.  ``all_scores``: the weights are the chosen experts' shares of the softmax over
    all experts (they do not add up to one); ``all_scores="sigmoid"``: the weight of a chosen expert is the sigmoid of its
    own logit, not renormalized; ``all_scores="steered"``: the experts are chosen by ``sigmoid(logit) + correction[e]``
    (``correction`` [experts] 32-bit or None) and a chosen expert's weight is ``weight_scale * sigmoid(logit)``."""
    _dev(logits, ids, weights, offsets, order, tiles, num_tiles)
    tokens, experts = logits.shape
    _f32s(logits, "moe_route: logits")      # rows may lie further apart than they are long (a view of some columns)
    _need(1 <= top <= min(experts, 64), f"moe_route: top {top} of {experts} experts")
    _i32(ids, offsets, order, tiles, num_tiles)
    _f32(weights, "moe_route: weights")
    _need(ids.numel() == tokens * top and weights.numel() == tokens * top and order.numel() == tokens * top
          and offsets.numel() == experts + 1 and tiles.numel() >= 2 * moe_max_tiles(tokens * top, experts, tile_rows)
          and num_tiles.numel() == 1 and tile_rows in (64, 128), "moe_route: output sizes")
    _need(1 <= keep <= groups <= 64 and experts % groups == 0 and (keep == groups or keep * (experts // groups) >= top),
          f"moe_route: {keep} of {groups} groups of {experts} experts for top {top}")
    mode = {"sigmoid": 2, "steered": 3}.get(all_scores, 1 if all_scores else 0)
    if correction is not None:
        _dev(correction)
        _need(mode == 3 and correction.dtype == torch.float32 and correction.is_contiguous()
              and correction.numel() == experts, "moe_route: one 32-bit correction per expert, with steered scores")
    fn = _fn("moe", "vk_moe_route_steered", [_p, _i, _i, _i, _i, _i, _i, _i, _p, _f, _ll, _p, _p, _p, _p, _p, _p, _p])
    _status(fn(_ptr(logits), experts, top, tokens, tile_rows, int(groups), int(keep), mode, _ptr(correction),
               float(weight_scale), logits.stride(0) if tokens > 1 else experts, _ptr(ids), _ptr(weights), _ptr(offsets),
               _ptr(order), _ptr(tiles), _ptr(num_tiles), _stream()), "moe_route")


def moe_experts(h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, offsets: torch.Tensor,
                order: torch.Tensor, tiles: torch.Tensor, num_tiles: torch.Tensor, weights: torch.Tensor, top: int,
                limit: float, alpha: float, act: torch.Tensor, pair_out: torch.Tensor, residual: torch.Tensor,
                accumulate: bool = True, weigh_input: bool = False) -> None:
    """The chosen experts of every token: ``y = g * sigmoid(alpha * g) * (u + 1)`` with ``g = min(Wg h, limit)`` and
    ``u = clamp(Wu h, -limit, limit)``, or with an infinite ``limit`` ``y = g * sigmoid(alpha * g) * u`` (alpha 1:
    ``silu(g) * u``); then ``Wd y``; ``residual += sum_j weights[t, j] * expert_j(h[t])`` (without ``accumulate``: ``=``).
    ``weigh_input``: ``residual += sum_j expert_j(weights[t, j] * h[t])`` instead."""
    _dev(h, w_gate, w_up, w_down, offsets, order, tiles, num_tiles, weights, act, pair_out, residual)
    tokens, width = h.shape
    experts, ff, _ = w_gate.shape
    _need(h.stride(1) == 1 and w_gate.shape == (experts, ff, width) and w_up.shape == w_gate.shape
          and w_down.shape == (experts, width, ff), "moe_experts: weight shapes")
    for t in (w_gate, w_up, w_down):
        _need(t.dtype == h.dtype and t.is_contiguous(), "moe_experts: weights must be contiguous and of h's dtype")
    _need(act.dtype == h.dtype and act.shape == (tokens * top, ff) and act.is_contiguous(), "moe_experts: act")
    _f32(pair_out, "moe_experts: pair_out")
    _f32(residual, "moe_experts: residual")
    _f32(weights, "moe_experts: weights")
    _need(pair_out.shape == (tokens * top, width) and residual.shape == (tokens, width) and weights.numel() == tokens * top,
          "moe_experts: output shapes")
    _i32(offsets, order, tiles, num_tiles)
    _need(offsets.numel() == experts + 1 and order.numel() == tokens * top
          and tiles.numel() >= 2 * moe_max_tiles(tokens * top, experts, moe_tile_rows(h, width, ff)),
          "moe_experts: grouping (made by moe_route with moe_tile_rows(h, width, ff))")
    fn = _fn("moe", "vk_moe_experts_weighed", [_p, _ll, _p, _p, _p, _i, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _f, _f, _p, _p,
                                               _p, _i, _i, _p])
    _status(fn(_ptr(h), h.stride(0), _ptr(w_gate), _ptr(w_up), _ptr(w_down), _dt(h, "h"), _ptr(offsets), _ptr(order),
               _ptr(tiles), _ptr(num_tiles), _ptr(weights), tokens, experts, top, width, ff, float(limit), float(alpha),
               _ptr(act), _ptr(pair_out), _ptr(residual), 1 if accumulate else 0, 1 if weigh_input else 0, _stream()),
            "moe_experts")


# --- norms behind a sublayer, sums of two streams, activations ------------------------------------------
def _f32s(tensor: torch.Tensor, what: str) -> None:
    """32-bit with unit inner stride; rows may lie further apart than they are long (a view of some columns)."""
    _need(tensor.dtype == torch.float32 and tensor.stride(-1) == 1, f"{what} must be float32 with a unit inner stride")


def rmsnorm_add(y: torch.Tensor, weight: torch.Tensor, eps: float, residual: torch.Tensor,
                next_out: Optional[torch.Tensor] = None, next_weight: Optional[torch.Tensor] = None,
                next_eps: float = 0.0) -> None:
    """``residual += y / sqrt(mean(y^2) + eps) * weight`` row by row, all 32-bit.  With ``next_out`` the new rows also
    leave as the next part's input, in its dtype: ``residual / sqrt(mean(residual^2) + next_eps) * next_weight`` (the
    norm in front of the next sublayer), or the rows as they are without ``next_weight``."""
    _dev(y, weight, residual, next_out, next_weight)
    _f32(y, "rmsnorm_add: y")
    _f32(residual, "rmsnorm_add: residual")
    rows, width = residual.shape
    _need(y.shape == residual.shape and y.is_contiguous() and residual.is_contiguous(), "rmsnorm_add: shapes")
    _need(weight.dtype == torch.float32 and weight.numel() == width and weight.is_contiguous(), "rmsnorm_add: weight")
    if next_out is not None:
        _need(next_out.shape == residual.shape and next_out.is_contiguous(), "rmsnorm_add: next_out")
    if next_weight is not None:
        _need(next_out is not None and next_weight.dtype == torch.float32 and next_weight.numel() == width
              and next_weight.is_contiguous(), "rmsnorm_add: next_weight")
    fn = _fn("elementwise", "vk_rmsnorm_add", [_p, _p, _p, _i, _i, _f, _p, _f, _p, _i, _p])
    _status(fn(_ptr(y), _ptr(weight), _ptr(residual), rows, width, float(eps), _ptr(next_weight), float(next_eps),
               _ptr(next_out), _dt(next_out, "next_out") if next_out is not None else 0, _stream()), "rmsnorm_add")


def axpby(x: torch.Tensor, a: float, y: torch.Tensor, b: float, out: torch.Tensor, accumulate: bool = False) -> None:
    """``out (+)= a * x + b * y``, elementwise, 32-bit."""
    _dev(x, y, out)
    for t, what in ((x, "x"), (y, "y"), (out, "out")):
        _f32(t, "axpby: " + what)
        _need(t.is_contiguous() and t.numel() == out.numel(), "axpby: three contiguous tensors of one size")
    fn = _fn("elementwise", "vk_axpby", [_p, _f, _p, _f, _p, _ll, _i, _p])
    _status(fn(_ptr(x), float(a), _ptr(y), float(b), _ptr(out), out.numel(), 1 if accumulate else 0, _stream()), "axpby")


ACTIVATIONS = {"none": 0, "relu2": 1, "silu": 2, "gelu_tanh": 3, "sigmoid": 4}


def activation(x: torch.Tensor, kind: str, out: torch.Tensor, mul: Optional[torch.Tensor] = None) -> None:
    """``out = act(x) (* mul)`` elementwise; ``x`` and ``mul`` may be row-strided views of either dtype, ``out`` is
    contiguous.  ``kind``: none (a change of type), relu2 (the square of relu), silu, gelu_tanh, sigmoid."""
    _dev(x, out, mul)
    _need(kind in ACTIVATIONS, f"activation: kind {kind!r}; known: {', '.join(ACTIVATIONS)}")
    rows, width = out.shape
    _need(x.shape == out.shape and x.stride(1) == 1 and out.is_contiguous(), "activation: shapes")
    if mul is not None:
        _need(mul.shape == out.shape and mul.stride(1) == 1, "activation: the factor's shape")
    fn = _fn("elementwise", "vk_activation", [_p, _i, _ll, _p, _i, _ll, _p, _i, _i, _i, _i, _p])
    _status(fn(_ptr(x), _dt(x, "x"), x.stride(0), _ptr(mul), _dt(mul, "mul") if mul is not None else 0,
               mul.stride(0) if mul is not None else 0, _ptr(out), _dt(out, "out"), rows, width, ACTIVATIONS[kind],
               _stream()), "activation")


def whole_norm_pack(proj: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                    heads: int, kv_heads: int, dim: int, vdim: int, padded: int, qkv: torch.Tensor) -> None:
    """From the 32-bit sums ``proj [T, >= q | k | v]``: q and k each divided by the root mean square of the whole
    projection (all heads at once) and multiplied by their weights (None: left as they are), and q, k and v laid out
    head by head, each padded with zeros to ``padded`` columns, as ``qkv [T, (heads + 2 kv_heads) * padded]``."""
    _dev(proj, q_weight, k_weight, qkv)
    _f32s(proj, "whole_norm_pack: proj")
    tokens = qkv.shape[0]
    need = (heads + kv_heads) * dim + kv_heads * vdim
    _need(proj.dim() == 2 and proj.shape[0] == tokens and proj.shape[1] >= need and proj.stride(1) == 1,
          "whole_norm_pack: proj")
    _need(padded >= max(dim, vdim) and qkv.shape == (tokens, (heads + 2 * kv_heads) * padded) and qkv.is_contiguous(),
          "whole_norm_pack: qkv")
    for weight, count in ((q_weight, heads * dim), (k_weight, kv_heads * dim)):
        if weight is not None:
            _need(weight.dtype == torch.float32 and weight.numel() == count and weight.is_contiguous(),
                  "whole_norm_pack: a weight per number of the projection")
    fn = _fn("elementwise", "vk_whole_norm_pack", [_p, _ll, _p, _p, _f, _i, _i, _i, _i, _i, _i, _p, _i, _p])
    _status(fn(_ptr(proj), proj.stride(0), _ptr(q_weight), _ptr(k_weight), float(eps), tokens, heads, kv_heads, dim, vdim,
               padded, _ptr(qkv), _dt(qkv, "qkv"), _stream()), "whole_norm_pack")


def head_norm_pack(proj: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                   heads: int, kv_heads: int, dim: int, vdim: int, padded: int, qkv: torch.Tensor,
                   first: Optional[torch.Tensor] = None, mix: Optional[torch.Tensor] = None) -> None:
    """From the 32-bit sums ``proj [T, >= q | k | v]``: every q head and every k head divided by its own root mean square
    and multiplied by a weight of ``dim`` numbers that the heads share (None: left as they are); with ``first`` (32-bit
    ``[T, kv_heads * vdim]``, row-strided) the values become ``(1 - mix) v + mix first``, ``mix`` one number on the
    device; q, k and v laid out head by head, each padded with zeros to ``padded`` columns."""
    _dev(proj, q_weight, k_weight, qkv, first, mix)
    _f32s(proj, "head_norm_pack: proj")
    tokens = qkv.shape[0]
    need = (heads + kv_heads) * dim + kv_heads * vdim
    _need(proj.dim() == 2 and proj.shape[0] == tokens and proj.shape[1] >= need and proj.stride(1) == 1,
          "head_norm_pack: proj")
    _need(padded >= max(dim, vdim) and qkv.shape == (tokens, (heads + 2 * kv_heads) * padded) and qkv.is_contiguous(),
          "head_norm_pack: qkv")
    for weight in (q_weight, k_weight):
        if weight is not None:
            _need(weight.dtype == torch.float32 and weight.numel() == dim and weight.is_contiguous(),
                  "head_norm_pack: a weight per number of a head")
    if first is not None:
        _need(first.dtype == torch.float32 and first.shape == (tokens, kv_heads * vdim) and first.stride(1) == 1,
              "head_norm_pack: first")
        _need(mix is not None and mix.dtype == torch.float32 and mix.numel() == 1, "head_norm_pack: mix must be one float32")
    fn = _fn("elementwise", "vk_head_norm_pack", [_p, _ll, _p, _p, _f, _p, _ll, _p, _i, _i, _i, _i, _i, _i, _p, _i, _p])
    _status(fn(_ptr(proj), proj.stride(0), _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(first),
               first.stride(0) if first is not None else 0, _ptr(mix) if first is not None else None, tokens, heads,
               kv_heads, dim, vdim, padded, _ptr(qkv), _dt(qkv, "qkv"), _stream()), "head_norm_pack")


def head_unpack_gate(attn: torch.Tensor, gate: Optional[torch.Tensor], gate_kind: str, heads: int, vdim: int,
                     padded: int, out: torch.Tensor) -> None:
    """``out[t, h * vdim + d] = attn[t, h * padded + d] * act(gate[t, h * vdim + d])``: the attention's output taken
    out of its padded heads and, with ``gate`` (32-bit, row-strided), gated."""
    _dev(attn, gate, out)
    tokens = out.shape[0]
    _need(attn.shape == (tokens, heads * padded) and attn.is_contiguous() and out.shape == (tokens, heads * vdim)
          and out.is_contiguous() and out.dtype == attn.dtype and padded >= vdim, "head_unpack_gate: shapes")
    _need(gate_kind in ACTIVATIONS, "head_unpack_gate: the gate's activation")
    if gate is not None:
        _f32s(gate, "head_unpack_gate: gate")
        _need(gate.shape == out.shape and gate.stride(1) == 1, "head_unpack_gate: gate")
    fn = _fn("elementwise", "vk_head_unpack_gate", [_p, _i, _p, _ll, _i, _i, _i, _i, _i, _p, _p])
    _status(fn(_ptr(attn), _dt(attn, "attn"), _ptr(gate), gate.stride(0) if gate is not None else 0,
               ACTIVATIONS[gate_kind], tokens, heads, vdim, padded, _ptr(out), _stream()), "head_unpack_gate")


# --- recurrences with a diagonal decay ------------------------------------------------------------------
DECAY_RULE_MAX_KEY_DIM = 256
SELECTIVE_SCAN_MAX_STATES = 256


def _lanes_share(n: int) -> int:
    return 1 if n <= 16 else 2 if n <= 32 else 4 if n <= 64 else 8 if n <= 128 else 16


def decay_rule_head_floats(dim: int, vdim: int) -> int:
    """Floats of one head's state as :func:`decay_rule` keeps it (the key channels padded)."""
    return vdim * 16 * _lanes_share(dim)


def selective_scan_channel_floats(states: int) -> int:
    """Floats of one channel's state as :func:`selective_scan` keeps it (padded)."""
    return 16 * _lanes_share(states)


def decay_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, silu_inputs: bool, decay: torch.Tensor,
               state: torch.Tensor, entry_start: torch.Tensor, entry_first_pos: torch.Tensor, slots: torch.Tensor,
               heads: int, dim: int, vdim: int, out: torch.Tensor, num_entries: int) -> None:
    """Linear attention with a fixed decay per head, ``S <- decay S + k v^T; o = S^T q``, over the step's entries in
    32-bit; ``q`` and ``k`` are row-strided views ``[T, heads * dim]`` with one stride, ``v [T, heads * vdim]``;
    ``silu_inputs``: all three pass through silu as they are read.  ``state [slots + 1, floats]`` starts with
    ``heads * decay_rule_head_floats(dim, vdim)`` floats of this layer."""
    _dev(q, k, v, decay, state, entry_start, entry_first_pos, slots, out)
    tokens = out.shape[0]
    for t, what in ((q, "q"), (k, "k"), (v, "v"), (decay, "decay"), (state, "state"), (out, "out")):
        _f32s(t, "decay_rule: " + what)
    _need(q.shape == (tokens, heads * dim) and k.shape == q.shape and q.stride(1) == 1 and k.stride(1) == 1
          and q.stride(0) == k.stride(0), "decay_rule: q and k")
    _need(v.shape == (tokens, heads * vdim) and v.stride(1) == 1 and out.shape == v.shape and out.is_contiguous(),
          "decay_rule: v and out")
    _need(decay.numel() == heads and decay.is_contiguous(), "decay_rule: a decay per head")
    _need(state.dim() == 2 and state.stride(1) == 1 and state.shape[1] >= heads * decay_rule_head_floats(dim, vdim),
          "decay_rule: state row too short")
    if dim > DECAY_RULE_MAX_KEY_DIM:
        raise UnsupportedError(f"decay_rule: a key width of {dim} is above the kernel's limit of {DECAY_RULE_MAX_KEY_DIM}")
    _i32(entry_start, entry_first_pos, slots)
    _entries_ok((entry_start, entry_first_pos, slots), num_entries)
    fn = _fn("scan", "vk_decay_rule", [_p, _p, _ll, _p, _ll, _i, _p, _p, _ll, _p, _p, _p, _i, _i, _i, _i, _p, _p])
    _status(fn(_ptr(q), _ptr(k), q.stride(0), _ptr(v), v.stride(0), 1 if silu_inputs else 0, _ptr(decay), _ptr(state),
               state.stride(0), _ptr(entry_start), _ptr(entry_first_pos), _ptr(slots), num_entries, heads, dim, vdim,
               _ptr(out), _stream()), "decay_rule")


def gated_norm(x: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, gate_kind: str, eps: float,
               out: torch.Tensor) -> None:
    """``out = x / rms(x) * weight * act(gate)`` over whole rows; ``x`` 32-bit, ``gate`` a 32-bit row-strided view."""
    _dev(x, weight, gate, out)
    _f32(x, "gated_norm: x")
    _f32s(gate, "gated_norm: gate")
    tokens, width = x.shape
    _need(x.is_contiguous() and out.shape == x.shape and out.is_contiguous() and gate.shape == x.shape
          and gate.stride(1) == 1, "gated_norm: shapes")
    _need(weight.dtype == torch.float32 and weight.numel() == width and weight.is_contiguous(), "gated_norm: weight")
    kinds = {"none": 0, "silu": 1, "sigmoid": 2}
    _need(gate_kind in kinds, "gated_norm: the gate's activation")
    fn = _fn("scan", "vk_gated_norm", [_p, _p, _p, _ll, _i, _f, _i, _i, _p, _i, _p])
    _status(fn(_ptr(x), _ptr(weight), _ptr(gate), gate.stride(0), kinds[gate_kind], float(eps), tokens, width, _ptr(out),
               _dt(out, "out"), _stream()), "gated_norm")


def causal_conv(x: torch.Tensor, conv: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
                conv_offset: int, entry_of: torch.Tensor, entry_start: torch.Tensor, entry_first_pos: torch.Tensor,
                slots: torch.Tensor, out32: torch.Tensor, out_run: Optional[torch.Tensor], num_entries: int) -> None:
    """``y[t, c] = silu(bias[c] + sum_j conv[c, j] x[t - (taps - 1 - j), c])`` per entry, with the inputs before the
    entry's first token from the state row (``(taps - 1) * C`` floats from ``conv_offset`` on; zeros at position 0),
    which afterwards holds the entry's last inputs.  ``x``: a 32-bit row-strided view ``[T, C]``; ``out32`` 32-bit
    and, if given, ``out_run`` the same in another dtype."""
    _dev(x, conv, bias, state, entry_of, entry_start, entry_first_pos, slots, out32, out_run)
    tokens, channels = out32.shape
    taps = conv.shape[1]
    _f32s(x, "causal_conv: x")
    _f32(conv, "causal_conv: conv")
    _f32s(state, "causal_conv: state")
    _f32(out32, "causal_conv: out32")
    _need(x.shape == (tokens, channels) and x.stride(1) == 1 and out32.is_contiguous(), "causal_conv: shapes")
    _need(conv.shape == (channels, taps) and conv.is_contiguous() and taps >= 1, "causal_conv: conv must be [C, taps]")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == channels and bias.is_contiguous(), "causal_conv: bias")
    if out_run is not None:
        _need(out_run.shape == out32.shape and out_run.is_contiguous(), "causal_conv: out_run")
    _need(state.dim() == 2 and state.stride(1) == 1 and conv_offset >= 0
          and state.shape[1] >= conv_offset + (taps - 1) * channels, "causal_conv: state row too short")
    _i32(entry_of, entry_start, entry_first_pos, slots)
    _need(entry_of.numel() >= tokens, "causal_conv: entry_of")
    _entries_ok((entry_start, entry_first_pos, slots), num_entries)
    fn = _fn("scan", "vk_causal_conv", [_p, _ll, _p, _p, _i, _i, _p, _ll, _ll, _p, _p, _p, _p, _i, _i, _p, _p, _i, _p])
    _status(fn(_ptr(x), x.stride(0), _ptr(conv), _ptr(bias), taps, channels, _ptr(state), state.stride(0), conv_offset,
               _ptr(entry_of), _ptr(entry_start), _ptr(entry_first_pos), _ptr(slots), tokens, num_entries, _ptr(out32),
               _ptr(out_run), _dt(out_run, "out_run") if out_run is not None else 0, _stream()), "causal_conv")


def selective_scan(x: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor, b: torch.Tensor, c: torch.Tensor,
                   a_log: torch.Tensor, skip: torch.Tensor, z: torch.Tensor, state: torch.Tensor,
                   entry_start: torch.Tensor, entry_first_pos: torch.Tensor, slots: torch.Tensor, out: torch.Tensor,
                   num_entries: int, prepared: bool = False) -> None:
    """The selective scan over the step's entries in 32-bit: per channel ``c`` and state ``n``
    ``step = softplus(dt + dt_bias); S <- exp(step * -exp(a_log)) S + step x b; y = S . c + skip x``, and
    ``out = y * silu(z)``.  ``x [T, C]`` contiguous; ``dt``, ``z`` row-strided views ``[T, C]``; ``b`` and ``c``
    row-strided views ``[T, N]`` of one buffer; ``state`` starts with ``C * selective_scan_channel_floats(N)`` floats.
    ``prepared``: ``dt`` already holds ``softplus(dt + dt_bias)`` and ``z`` already ``silu(z)`` (:func:`scan_prepare`)."""
    _dev(x, dt, dt_bias, b, c, a_log, skip, z, state, entry_start, entry_first_pos, slots, out)
    tokens, channels = x.shape
    states = a_log.shape[1]
    for t, what in ((x, "x"), (dt, "dt"), (dt_bias, "dt_bias"), (b, "b"), (c, "c"), (a_log, "a_log"), (skip, "skip"),
                    (z, "z"), (state, "state")):
        _f32s(t, "selective_scan: " + what)
    _need(x.is_contiguous() and dt.shape == x.shape and dt.stride(1) == 1 and z.shape == x.shape and z.stride(1) == 1
          and out.shape == x.shape and out.is_contiguous(), "selective_scan: x, dt, z, out")
    _need(b.shape == (tokens, states) and c.shape == b.shape and b.stride(1) == 1 and c.stride(1) == 1
          and b.stride(0) == c.stride(0), "selective_scan: b and c")
    _need(a_log.shape == (channels, states) and a_log.is_contiguous() and dt_bias.numel() == channels
          and dt_bias.is_contiguous() and skip.numel() == channels and skip.is_contiguous(), "selective_scan: parameters")
    if states > SELECTIVE_SCAN_MAX_STATES:
        raise UnsupportedError(f"selective_scan: {states} states a channel are above the kernel's limit of "
                               f"{SELECTIVE_SCAN_MAX_STATES}")
    _need(state.dim() == 2 and state.stride(1) == 1
          and state.shape[1] >= channels * selective_scan_channel_floats(states), "selective_scan: state row too short")
    _i32(entry_start, entry_first_pos, slots)
    _entries_ok((entry_start, entry_first_pos, slots), num_entries)
    fn = _fn("scan", "vk_selective_scan", [_p, _p, _ll, _p, _p, _p, _ll, _p, _p, _p, _ll, _p, _ll, _p, _p, _p, _i, _i, _i,
                                           _i, _p, _i, _p])
    _status(fn(_ptr(x), _ptr(dt), dt.stride(0), _ptr(dt_bias), _ptr(b), _ptr(c), b.stride(0), _ptr(a_log), _ptr(skip),
               _ptr(z), z.stride(0), _ptr(state), state.stride(0), _ptr(entry_start), _ptr(entry_first_pos), _ptr(slots),
               num_entries, channels, states, 1 if prepared else 0, _ptr(out), _dt(out, "out"), _stream()),
            "selective_scan")


def scan_prepare(dt: torch.Tensor, dt_bias: torch.Tensor, z: torch.Tensor, gate: torch.Tensor) -> None:
    """``dt <- softplus(dt + dt_bias)`` in place and ``gate = silu(z)``, for :func:`selective_scan` with ``prepared``: a
    prompt's portion takes them once for all its tokens instead of token behind token inside the recurrence."""
    _dev(dt, dt_bias, z, gate)
    tokens, channels = gate.shape
    for t, what in ((dt, "dt"), (z, "z")):
        _f32s(t, "scan_prepare: " + what)
        _need(t.shape == gate.shape, "scan_prepare: shapes")
    _f32(gate, "scan_prepare: gate")
    _need(dt_bias.dtype == torch.float32 and dt_bias.numel() == channels and dt_bias.is_contiguous(), "scan_prepare: dt_bias")
    fn = _fn("scan", "vk_scan_prepare", [_p, _ll, _p, _p, _ll, _p, _i, _i, _p])
    _status(fn(_ptr(dt), dt.stride(0), _ptr(dt_bias), _ptr(z), z.stride(0), _ptr(gate), tokens, channels, _stream()),
            "scan_prepare")


# ----------------------------------------------------------------------------------------------
_GATE_ACTS = {"none": 0, "silu": 2, "sigmoid": 4}


def head_prepare(proj: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], norm: bool,
                 norm_first: bool, eps: float, positions: Optional[torch.Tensor], inv_freq: Optional[torch.Tensor],
                 rot_dims: int, heads: int, kv_heads: int, maps: int, dim: int, vdim: int, width: int,
                 qkv: torch.Tensor, k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None,
                 entry_of_token: Optional[torch.Tensor] = None, block_table: Optional[torch.Tensor] = None) -> None:
    """The 32-bit sums ``proj`` = ``[q | k | v | ...]`` of a step's tokens laid out head by head at one padded
    ``width`` in ``qkv``: q and k heads rotated by position (the first ``rot_dims`` numbers, half-split pairs) and, with
    ``norm``, divided by their root mean square and multiplied by a weight of ``dim`` numbers (None: no weight), before
    the rotation (``norm_first``) or behind it.  ``maps`` > 1: that many attention maps per head; a query head's maps
    become query heads of their own, each in its own columns of the padded width, and a key head's maps stay side by
    side in one key head, so every map meets its own keys and all maps of a head read the same values.  With
    ``k_cache`` (``[pages, kv_heads, block_size, width]``), ``v_cache`` (transposed), ``entry_of_token`` and
    ``block_table``: the tokens' key and value heads also go into their pages, as :func:`rope_kvwrite` would put them."""
    _dev(proj, q_weight, k_weight, positions, inv_freq, qkv, k_cache, v_cache, entry_of_token, block_table)
    tokens = proj.shape[0]
    need = (heads + kv_heads) * maps * dim + kv_heads * vdim
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= need,
          "head_prepare: proj must be 32-bit [tokens, >= q + k + v columns]")
    _need(qkv.shape == (tokens, (heads * maps + 2 * kv_heads) * width) and qkv.is_contiguous(), "head_prepare: qkv shape")
    _need(width >= maps * dim and width >= vdim and dim <= 256, "head_prepare: the padded width holds every head")
    for weight in (q_weight, k_weight):
        if weight is not None:
            _need(weight.dtype == torch.float32 and weight.numel() == dim and weight.is_contiguous(), "head_prepare: weights")
    if rot_dims:
        _need(rot_dims % 2 == 0 and rot_dims <= dim and positions is not None and positions.dtype == torch.int32
              and positions.numel() >= tokens and inv_freq is not None and inv_freq.dtype == torch.float32
              and inv_freq.numel() == rot_dims // 2, "head_prepare: rotation operands")
    table_width = block_size = 0
    if k_cache is not None:
        _need(v_cache is not None and block_table is not None and entry_of_token is not None and positions is not None,
              "head_prepare: a cache needs its table, the tokens' entries and their positions")
        _need(_cache_ok(k_cache, v_cache, kv_heads, width, qkv.dtype), "head_prepare: cache shape or dtype")
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
              "head_prepare: block table")
        _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() >= tokens and positions.dtype == torch.int32
              and positions.numel() >= tokens, "head_prepare: entries and positions")
        table_width, block_size = block_table.shape[1], k_cache.shape[2]
    fn = _fn("heads", "vk_head_prepare", [_p, _ll, _p, _p, _i, _i, _f, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p, _i,
                                          _p, _p, _p, _p, _i, _i, _p])
    _status(fn(_ptr(proj), proj.stride(0), _ptr(q_weight), _ptr(k_weight), 1 if norm else 0, 1 if norm_first else 0,
               float(eps), _ptr(positions), _ptr(inv_freq), int(rot_dims), tokens, heads, kv_heads, maps, dim, vdim,
               width, _ptr(qkv), _dt(qkv, "qkv"), _ptr(k_cache), _ptr(v_cache), _ptr(entry_of_token), _ptr(block_table),
               table_width, block_size, _stream()), "head_prepare")


def head_finish(attn: torch.Tensor, out: torch.Tensor, heads: int, vdim: int, width: int, maps: int = 1,
                subtract: float = 0.0, unit_norm: bool = False, eps: float = 0.0, factor: float = 1.0,
                gate: Optional[torch.Tensor] = None, gate_kind: str = "none", gate_per_head: bool = False) -> None:
    """The attention kernels' output (``heads * maps`` heads of padded ``width``) becomes the output product's input
    ``out [tokens, heads * vdim]``: with two maps ``a_1 - subtract * a_2``; with ``unit_norm`` divided by the head's
    root mean square; times ``factor``; times ``gate_kind(gate)``, one 32-bit number per head (``gate_per_head``,
    ``gate [tokens, >= heads]``) or per number (``gate [tokens, >= heads * vdim]``)."""
    _dev(attn, out, gate)
    tokens = attn.shape[0]
    _need(attn.shape == (tokens, heads * maps * width) and attn.is_contiguous() and maps in (1, 2), "head_finish: attn shape")
    _need(out.shape == (tokens, heads * vdim) and out.is_contiguous() and out.dtype == attn.dtype, "head_finish: out shape")
    _need(vdim <= width and vdim <= 256, "head_finish: widths")
    _need(gate_kind in _GATE_ACTS, f"head_finish: gate {gate_kind!r}")
    ldg = 0
    if gate is not None:
        _need(gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == tokens and gate.stride(1) == 1
              and gate.shape[1] >= (heads if gate_per_head else heads * vdim), "head_finish: gate shape")
        ldg = gate.stride(0)
    fn = _fn("heads", "vk_head_finish", [_p, _i, _i, _f, _i, _f, _f, _p, _ll, _i, _i, _i, _i, _i, _i, _p, _p])
    _status(fn(_ptr(attn), _dt(attn, "attn"), maps, float(subtract), 1 if unit_norm else 0, float(eps), float(factor),
               _ptr(gate), ldg, 1 if gate_per_head else 0, _GATE_ACTS[gate_kind], tokens, heads, vdim, width, _ptr(out),
               _stream()), "head_finish")


def rotate_scale(x: torch.Tensor, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rot_dims: int, heads: int,
                 dim: int, factor: float = 1.0) -> None:
    """``heads`` heads of ``dim`` 32-bit numbers from column 0 of ``x`` (rows may be strided) rotated in place by their
    token's position (the first ``rot_dims`` numbers, half-split pairs) and multiplied by ``factor``."""
    _dev(x, positions, inv_freq)
    tokens = x.shape[0]
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1 and x.shape[1] >= heads * dim, "rotate_scale: x")
    _need(rot_dims % 2 == 0 and 0 <= rot_dims <= dim, "rotate_scale: rot_dims")
    if rot_dims:
        _need(positions.dtype == torch.int32 and positions.numel() >= tokens and inv_freq is not None
              and inv_freq.dtype == torch.float32 and inv_freq.numel() == rot_dims // 2, "rotate_scale: rotation operands")
    fn = _fn("heads", "vk_rotate_scale", [_p, _ll, _p, _p, _i, _i, _i, _i, _f, _p])
    _status(fn(_ptr(x), x.stride(0), _ptr(positions), _ptr(inv_freq), int(rot_dims), tokens, heads, dim, float(factor),
               _stream()), "rotate_scale")


def row_gate_add(y: torch.Tensor, gate: torch.Tensor, gate_kind: str, out: torch.Tensor, accumulate: bool = True) -> None:
    """``out[r, :] (+)= gate_kind(gate[r]) * y[r, :]``: 32-bit rows gated by one number each (``gate [rows, >= 1]``)."""
    _dev(y, gate, out)
    _need(y.dtype == torch.float32 and out.dtype == torch.float32 and y.shape == out.shape and y.dim() == 2
          and y.is_contiguous() and out.is_contiguous(), "row_gate_add: two contiguous 32-bit matrices of one shape")
    _need(gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == y.shape[0], "row_gate_add: gate")
    _need(gate_kind in _GATE_ACTS, f"row_gate_add: gate {gate_kind!r}")
    fn = _fn("heads", "vk_row_gate_add", [_p, _p, _ll, _i, _p, _i, _i, _i, _p])
    _status(fn(_ptr(y), _ptr(gate), gate.stride(0), _GATE_ACTS[gate_kind], _ptr(out), y.shape[0], y.shape[1],
               1 if accumulate else 0, _stream()), "row_gate_add")
