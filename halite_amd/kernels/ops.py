"""Typed Python wrappers of the kernel library's entry points.

Each wrapper checks on the host what its kernel assumes (device, dtype, layout,
shapes) before it launches on torch's current stream; a failed check or a failed
launch raises ``KernelError``.  There is no other implementation behind these
functions: without a GPU and the built library they raise.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass

import torch

from . import library

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


@dataclass
class NextNorm:
    """What a part's last product is told about the RMSNorm that reads its result: the
    float32 residual stream the result is added into, and the norm's weight and eps."""

    h: torch.Tensor
    weight: torch.Tensor
    eps: float


@dataclass
class NormedRows:
    """At most 32 rows on their way through an RMSNorm whose scaling is left to the product
    that reads them: ``x`` [rows, d] is ``bf16(weight * bf16(h))`` and ``ss_parts``
    [parts, 16 or 32] holds partial sums of ``h^2`` per row, so the norm's output is
    ``x * rsqrt(ss_parts.sum(0) / d + eps)`` row by row."""

    x: torch.Tensor
    ss_parts: torch.Tensor
    eps: float
    weight: torch.Tensor  # of the norm the rows were prepared for

    @property
    def shape(self):
        return self.x.shape

    @property
    def dtype(self):
        return self.x.dtype

    def materialize(self) -> torch.Tensor:
        """The norm's output as a tensor, for a reader that does not scale by itself."""
        lib = library.core_library()
        x, ss = self.x, self.ss_parts
        _dev(ss)
        _need(x.is_cuda and x.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1, "normed rows are bf16 rows")
        _need(ss.dtype == torch.float32 and ss.dim() == 2, "sums of squares are float32 [parts, rows]")
        m, d = x.shape
        out = torch.empty((m, d), dtype=torch.bfloat16, device=x.device)
        _check(lib, lib.hal_scale_normed_rows(
            _ptr(x), x.stride(0), _ptr(ss), ss.shape[0], ss.shape[1], ctypes.c_float(self.eps), _ptr(out), m, d, _stream()))
        return out


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dtype}") from None


def _ptr(t: torch.Tensor | None):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, msg: str):
    if not cond:
        raise KernelError(msg)


def _dev(*tensors):
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel arguments must be on the GPU")
            _need(t.is_contiguous(), "kernel arguments must be contiguous")


def _check(lib, rc: int):
    if rc != 0:
        raise KernelError(lib.hal_last_error().decode())


def _i32(t: torch.Tensor | None, name: str):
    if t is not None:
        _need(t.dtype == torch.int32, f"{name} must be int32")


# --------------------------------------------------------------------------------


def embedding(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor | None = None):
    """``out[t] = table[ids[t]]`` as float32."""
    lib = library.core_library()
    _dev(ids, table, out)
    _i32(ids, "ids")
    n, (vocab, d) = ids.numel(), table.shape
    if out is None:
        out = torch.empty((n, d), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (n, d), "embedding: bad output")
    _check(
        lib,
        lib.hal_embedding(_ptr(ids), _ptr(table), dtype_code(table.dtype), _ptr(out), n, d, vocab, _stream()),
    )
    return out


def take_tokens(src: torch.Tensor, tokens: torch.Tensor) -> None:
    """``tokens[i] = src[tokens[i]]`` in place: token ids that an earlier step left on the
    device go into a step's array without a round over the host."""
    lib = library.core_library()
    _dev(src, tokens)
    _i32(src, "src")
    _i32(tokens, "tokens")
    _check(lib, lib.hal_take_tokens(_ptr(src), src.numel(), _ptr(tokens), tokens.numel(), _stream()))


def rmsnorm(
    h: torch.Tensor,
    weight: torch.Tensor,
    eps: float,
    out_dtype: torch.dtype,
    delta: torch.Tensor | None = None,
    rows: torch.Tensor | None = None,
    update_h: bool = True,
):
    """RMSNorm of the float32 stream ``h`` (+ ``delta``), optionally only of
    ``rows``; with ``delta`` and ``update_h`` the sum is written back to ``h``."""
    lib = library.core_library()
    _dev(h, weight, delta, rows)
    _i32(rows, "rows")
    _need(h.dtype == torch.float32 and h.dim() == 2, "rmsnorm: the stream is float32 [T, d]")
    n_tokens, d = h.shape
    _need(weight.shape == (d,), f"rmsnorm: weight {tuple(weight.shape)} for width {d}")
    if delta is not None:
        _need(delta.shape == h.shape and delta.dtype == out_dtype, "rmsnorm: bad delta")
    n_rows = n_tokens if rows is None else rows.numel()
    if rows is not None:
        update_h = False
    out = torch.empty((n_rows, d), dtype=out_dtype, device=h.device)
    _check(
        lib,
        lib.hal_rmsnorm(
            _ptr(h), _ptr(delta), _ptr(rows), _ptr(weight), dtype_code(weight.dtype),
            ctypes.c_float(eps), _ptr(out), dtype_code(out_dtype), n_rows, d,
            1 if (update_h and delta is not None) else 0, _stream(),
        ),
    )
    return out


def residual_add(h: torch.Tensor, delta: torch.Tensor):
    lib = library.core_library()
    _dev(h, delta)
    _need(h.dtype == torch.float32 and delta.shape == h.shape, "residual_add: bad shapes")
    _check(
        lib,
        lib.hal_residual_add(_ptr(h), _ptr(delta), dtype_code(delta.dtype), ctypes.c_longlong(h.numel()), _stream()),
    )
    return h


def silu_mul(gate_up: torch.Tensor):
    """``up * silu(gate)`` of rows ``[gate | up]``."""
    lib = library.core_library()
    _dev(gate_up)
    n, two_f = gate_up.shape
    _need(two_f % 2 == 0, "silu_mul: odd row length")
    out = torch.empty((n, two_f // 2), dtype=gate_up.dtype, device=gate_up.device)
    _check(
        lib,
        lib.hal_silu_mul(_ptr(gate_up), _ptr(out), dtype_code(gate_up.dtype), n, two_f // 2, _stream()),
    )
    return out


def rope_append(
    qkv: torch.Tensor,
    positions: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    n_heads: int,
    n_kv_heads: int,
    head_dim: int,
    rotary_dim: int,
    interleaved: bool,
    token_seg: torch.Tensor | None = None,
    block_table: torch.Tensor | None = None,
    k_pages: torch.Tensor | None = None,
    v_pages: torch.Tensor | None = None,
    page_size: int = 0,
    tiled: bool = False,
):
    """Rotate q and k in place in the packed rows ``[q | k | v]`` and append k and
    v to the pages (``n_kv_heads == 0``: rows hold q only, nothing is appended);
    ``tiled`` says that the pages are kept in the matrix-core kernel's own order."""
    lib = library.core_library()
    _dev(qkv, positions, cos, sin, token_seg, block_table, k_pages, v_pages)
    _i32(positions, "positions"), _i32(token_seg, "token_seg"), _i32(block_table, "block_table")
    n = qkv.shape[0]
    _need(positions.numel() == n, "rope_append: one position per row")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32, "rope tables are float32")
    _need(rotary_dim == 0 or (cos.shape[1] == rotary_dim // 2 and cos.shape == sin.shape), "rope table width")
    n_pages = 0
    if n_kv_heads > 0:
        _need(k_pages is not None and v_pages is not None and block_table is not None, "rope_append: no cache")
        _need(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "cache dtype != activation dtype")
        n_pages = k_pages.shape[0]
        _need(
            k_pages.shape == (n_pages, n_kv_heads, page_size, head_dim)
            and v_pages.shape == (n_pages, n_kv_heads, head_dim, page_size),
            "rope_append: page shapes",
        )
        _need(token_seg.numel() == n and block_table.dim() == 2, "rope_append: segment arrays")
    _check(
        lib,
        lib.hal_rope_append(
            _ptr(qkv), dtype_code(qkv.dtype), qkv.shape[1], _ptr(positions), _ptr(token_seg),
            _ptr(block_table), 0 if block_table is None else block_table.shape[1],
            _ptr(cos), _ptr(sin), cos.shape[0], _ptr(k_pages), _ptr(v_pages),
            n, n_heads, n_kv_heads, head_dim, rotary_dim, 1 if interleaved else 0,
            page_size, n_pages, 1 if tiled else 0, _stream(),
        ),
    )


def pair_rows_for_rotation(w_qkv: torch.Tensor, head_dim: int) -> torch.Tensor:
    """The packed q, k, v weight with the rows of every head reordered to
    ``[8j .. 8j+7, D/2 + 8j .. D/2 + 8j+7]`` for ``j = 0 .. D/16 - 1``, so that a tile of
    16 rows holds eight rotation pairs ``(d, d + D/2)``: the order ``qkv_rope_append``
    takes (after ``tile_weight``)."""
    n, _ = w_qkv.shape
    _need(head_dim % 16 == 0 and n % head_dim == 0, "pair_rows_for_rotation: head size in steps of 16")
    within = torch.arange(head_dim, device=w_qkv.device).view(2, head_dim // 16, 8).permute(1, 0, 2).reshape(-1)
    heads = torch.arange(n // head_dim, device=w_qkv.device) * head_dim
    return w_qkv[(heads[:, None] + within[None, :]).reshape(-1)]


def qkv_rope_append(
    x: torch.Tensor,
    w_paired_tiled: torch.Tensor,
    positions: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    n_heads: int,
    n_kv_heads: int,
    head_dim: int,
    token_seg: torch.Tensor,
    block_table: torch.Tensor,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    page_size: int,
    tiled: bool = False,
) -> torch.Tensor:
    """The packed q, k, v projection of at most 16 bf16 rows, the rotation of q and k
    (pairs ``(j, j + D/2)``, the whole head) and the append of k and v to the pages, in
    one kernel.  ``w_paired_tiled`` is ``tile_weight(pair_rows_for_rotation(w_qkv, D))``;
    ``x`` may be ``NormedRows``, whose scaling the kernel then applies.
    Returns the rotated queries ``[rows, n_heads * head_dim]``."""
    lib = library.core_library()
    normed = x if isinstance(x, NormedRows) else None
    if normed is not None:
        x = normed.x
    _dev(x, w_paired_tiled, positions, cos, sin, token_seg, block_table, k_pages, v_pages)
    _i32(positions, "positions"), _i32(token_seg, "token_seg"), _i32(block_table, "block_table")
    m, k = x.shape
    n = (n_heads + 2 * n_kv_heads) * head_dim
    _need(x.dtype == torch.bfloat16 and x.stride(1) == 1 and m <= FUSED_ROWS, "qkv_rope_append: up to 32 bf16 rows")
    _need(normed is None or (normed.ss_parts.shape[1] == 16 * -(-m // 16) and normed.ss_parts.is_contiguous()),
          "qkv_rope_append: sums of squares")
    _need(head_dim % 16 == 0 and k % 8 == 0, "qkv_rope_append: head size in steps of 16, width in steps of 8")
    _need(
        w_paired_tiled.dtype == torch.bfloat16 and w_paired_tiled.is_contiguous()
        and w_paired_tiled.numel() == n * (-(-k // 32) * 32),
        "qkv_rope_append: tiled weight",
    )
    _need(positions.numel() == m and token_seg.numel() == m and block_table.dim() == 2, "qkv_rope_append: step arrays")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape
          and cos.dim() == 2 and cos.shape[1] == head_dim // 2 and cos.is_contiguous() and sin.is_contiguous(),
          "qkv_rope_append: rotation tables")
    n_pages = k_pages.shape[0]
    _need(k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16
          and k_pages.shape == (n_pages, n_kv_heads, page_size, head_dim)
          and v_pages.shape == (n_pages, n_kv_heads, head_dim, page_size), "qkv_rope_append: pages")
    q = torch.empty((m, n_heads * head_dim), dtype=torch.bfloat16, device=x.device)
    _check(
        lib,
        lib.hal_qkv_rope_append(
            _ptr(x), x.stride(0), _ptr(w_paired_tiled), _ptr(q), m, k, _ptr(positions), _ptr(token_seg),
            _ptr(block_table), block_table.shape[1], _ptr(cos), _ptr(sin), cos.shape[0],
            _ptr(k_pages), _ptr(v_pages), n_heads, n_kv_heads, head_dim, page_size, n_pages,
            1 if tiled else 0, _ptr(normed.ss_parts) if normed else None,
            normed.ss_parts.shape[0] if normed else 0, ctypes.c_float(normed.eps if normed else 0.0),
            _stream(),
        ),
    )
    return q


def attention_simple(
    q: torch.Tensor,
    q_row_stride: int,
    positions: torch.Tensor,
    token_seg: torch.Tensor,
    block_table: torch.Tensor,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    n_heads: int,
    scale: float,
    window: int = 0,
    max_kv_len: int | None = None,
    min_q_len: int = 1,
):
    """Paged attention in float32 arithmetic; ``q`` holds the query heads at the start of
    rows of ``q_row_stride`` elements.  ``max_kv_len``: the most keys that a request of the
    step has (what the block table could hold if it is not given); ``min_q_len``: the fewest
    tokens that a request has in the step (1 if not known: steps of prompts alone go to the
    matrix cores).  They decide how the step is cut into workgroups, never a result."""
    lib = library.core_library()
    _dev(q, positions, token_seg, block_table, k_pages, v_pages)
    _i32(positions, "positions"), _i32(token_seg, "token_seg"), _i32(block_table, "block_table")
    n = positions.numel()
    n_pages, n_kv, page_size, head_dim = k_pages.shape
    _need(v_pages.shape == (n_pages, n_kv, head_dim, page_size), "attention: page shapes")
    _need(k_pages.dtype == q.dtype and v_pages.dtype == q.dtype, "attention: cache dtype")
    _need(q.numel() >= n * q_row_stride and q_row_stride >= n_heads * head_dim, "attention: q rows")
    out = torch.empty((n, n_heads * head_dim), dtype=q.dtype, device=q.device)
    if max_kv_len is None:
        max_kv_len = block_table.shape[1] * page_size
    tq, split, rows, pieces, floats = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_longlong()
    _check(lib, lib.hal_attention_simple_plan(n, n_heads, n_kv, head_dim, max_kv_len, min_q_len, ctypes.byref(tq),
                                              ctypes.byref(split), ctypes.byref(rows), ctypes.byref(pieces),
                                              ctypes.byref(floats)))
    part = torch.empty(floats.value, dtype=torch.float32, device=q.device) if floats.value else None
    _check(
        lib,
        lib.hal_attention_simple(
            _ptr(q), q_row_stride, _ptr(out), n_heads * head_dim, dtype_code(q.dtype),
            _ptr(positions), _ptr(token_seg), _ptr(block_table), block_table.shape[1],
            _ptr(k_pages), _ptr(v_pages), _ptr(part), n, n_heads, n_kv, head_dim, page_size, n_pages,
            ctypes.c_float(scale), window, max_kv_len, min_q_len, _stream(),
        ),
    )
    return out


def gemm_f32(a: torch.Tensor, w: torch.Tensor):
    """``a @ w.T`` in true float32 (``a`` [M, K], ``w`` [N, K])."""
    lib = library.core_library()
    _dev(a, w)
    _need(a.dtype == torch.float32 and w.dtype == torch.float32, "gemm_f32 takes float32")
    m, k = a.shape
    n, k2 = w.shape
    _need(k == k2, f"gemm_f32: inner sizes {k} and {k2}")
    out = torch.empty((m, n), dtype=torch.float32, device=a.device)
    _check(lib, lib.hal_gemm_f32(_ptr(a), k, _ptr(w), k, _ptr(out), n, m, n, k, _stream()))
    return out


def sample(
    logits: torch.Tensor,
    temperature: torch.Tensor,
    top_k: torch.Tensor,
    top_p: torch.Tensor,
    min_p: torch.Tensor,
    seeds: torch.Tensor,
    draw_index: torch.Tensor,
    all_greedy: bool = False,
    key_scratch: bool = True,
    unfiltered: bool = False,
    spread: bool = False,
    late: bool = True,
):
    """Next token and log-probability of every row of float32 ``logits``.
    ``all_greedy`` promises that no row samples (``temperature`` 0 or ``top_k`` 1 in
    every row), ``unfiltered`` that every row is greedy or draws from its whole
    distribution (no top-k, top-p or min-p): the rows are then spread over many blocks,
    in two launches.  ``spread``: every pass over a row is shared by 32 blocks (ten
    launches; seven more unless ``late`` is false, which promises that no row has top-k,
    top-p and min-p all at once).  Otherwise, with
    ``key_scratch``, the kernel gets room for one 32-bit key per logit, which its passes
    over a row read instead of deriving it again."""
    lib = library.core_library()
    _dev(logits, temperature, top_k, top_p, min_p, seeds, draw_index)
    n, vocab = logits.shape
    _need(logits.dtype == torch.float32, "sample: logits are float32")
    _need(temperature.dtype == torch.float32 and top_p.dtype == torch.float32 and min_p.dtype == torch.float32, "sample: float parameters")
    _i32(top_k, "top_k"), _i32(draw_index, "draw_index")
    _need(seeds.dtype == torch.int64, "sample: seeds are int64")
    for t in (temperature, top_k, top_p, min_p, seeds, draw_index):
        _need(t.numel() == n, "sample: one parameter per row")
    # one buffer for both results, so that the host can fetch them with one copy
    both = torch.empty(2 * n, dtype=torch.int32, device=logits.device)
    tokens, logprobs = both[:n], both[n:].view(torch.float32)
    if all_greedy and logits.is_contiguous():  # every row spread over many blocks
        parts = torch.empty((n, 32, 4), dtype=torch.float32, device=logits.device)
        _check(lib, lib.hal_sample_greedy(_ptr(logits), vocab, n, vocab, _ptr(parts), _ptr(tokens), _ptr(logprobs), _stream()))
        return tokens, logprobs
    if unfiltered and logits.is_contiguous():
        parts = torch.empty((n, 32, 4), dtype=torch.float32, device=logits.device)
        _check(lib, lib.hal_sample_unfiltered(
            _ptr(logits), vocab, n, vocab, _ptr(temperature), _ptr(top_k), _ptr(seeds), _ptr(draw_index),
            _ptr(parts), _ptr(tokens), _ptr(logprobs), _stream()))
        return tokens, logprobs
    if spread and logits.is_contiguous():
        dev = logits.device
        parts = torch.empty((n, 32, 4), dtype=torch.float32, device=dev)
        kept = torch.empty((n, 32), dtype=torch.float32, device=dev)
        state = torch.empty((n, 20), dtype=torch.int32, device=dev)
        hist = torch.empty((n, 2, 2048), dtype=torch.int64, device=dev)
        _check(lib, lib.hal_sample_spread(
            _ptr(logits), vocab, n, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(min_p),
            _ptr(seeds), _ptr(draw_index), _ptr(parts), _ptr(kept), _ptr(state), _ptr(hist),
            1 if late else 0, _ptr(tokens), _ptr(logprobs), _stream()))
        return tokens, logprobs
    keys = torch.empty((n, vocab), dtype=torch.int32, device=logits.device) if key_scratch and not all_greedy else None
    _check(
        lib,
        lib.hal_sample(
            _ptr(logits), vocab, n, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(min_p),
            _ptr(seeds), _ptr(draw_index), _ptr(tokens), _ptr(logprobs), _ptr(keys), _stream(),
        ),
    )
    return tokens, logprobs


SKINNY_MAX_ROWS = 64  # what the kernel takes
SKINNY_ROWS = 16  # up to here it beats the library product
FUSED_ROWS = 32  # what the epilogues that take other kernels' work take
FUSED_MID_ELEMENTS = 32 * 1024 * 1024  # the largest matrix on which they pay at 17 to 32 rows
GATED_MID_ELEMENTS = 64 * 1024 * 1024  # the same for the gated product with SiLU*mul (each of its two matrices)
# ... if the weights lie in its tiled order.  On row-major weights (a model too large for
# the second copy) it wins only on small matrices or a single row: measured on Llama-3.1-70B
# shapes at 8 and 16 rows, the library reads 4.7-5.5 TB/s where the kernel reads 3.2-4.6.
ROW_MAJOR_SKINNY_ELEMENTS = 32 * 1024 * 1024


def skinny_pays(m: int, n: int, k: int, tiled: bool) -> bool:
    """Whether the small-batch kernel is the faster way for ``m`` rows against an
    ``[n, k]`` bf16 weight."""
    if m > SKINNY_ROWS:
        return False
    return tiled or m == 1 or n * k <= ROW_MAJOR_SKINNY_ELEMENTS
_MM_OUT_DTYPE = None  # whether torch.mm takes out_dtype (found at first use)


def tile_weight(w: torch.Tensor) -> torch.Tensor:
    """``w`` [N, K] in the small-batch kernel's own order: [16-row tile][32-column
    step][lane][8 elements], zero-padded, where lane ``l`` of a tile holds row
    ``l % 16`` and columns ``(l // 16) * 8 ...`` of the step.  A wave's load then reads
    one contiguous KiB."""
    n, k = w.shape
    n_pad, k_pad = -(-n // 16) * 16, -(-k // 32) * 32
    if (n_pad, k_pad) != (n, k):
        padded = torch.zeros((n_pad, k_pad), dtype=w.dtype, device=w.device)
        padded[:n, :k] = w
        w = padded
    t = w.view(n_pad // 16, 16, k_pad // 32, 4, 8).permute(0, 2, 3, 1, 4)
    return t.contiguous().view(-1)


def gemm_bf16_skinny(
    x: torch.Tensor,
    w: torch.Tensor,
    w_up: torch.Tensor | None = None,
    out_dtype: torch.dtype = torch.bfloat16,
    add_to: torch.Tensor | None = None,
    tiled_shape: tuple[int, int] | None = None,
):
    """``x @ w.T`` for at most 64 rows of bf16 ``x``; with ``w_up`` the gated form
    ``(x @ w_up.T) * silu(x @ w.T)``; ``add_to`` (float32) receives ``+=``."""
    lib = library.core_library()
    _dev(x, add_to)
    _need(x.dtype == torch.bfloat16, "skinny gemm takes bf16")
    m, k = x.shape
    if tiled_shape is not None:  # weights from tile_weight()
        n, k2 = tiled_shape
        need = (-(-n // 16) * 16) * (-(-k2 // 32) * 32)
        for t in (w, w_up):
            if t is not None:
                _need(t.is_cuda and t.dtype == torch.bfloat16 and t.numel() == need and t.is_contiguous(), "skinny gemm: tiled weight")
        ldw = 0
    else:
        for t in (w, w_up):
            if t is not None:
                _need(t.is_cuda and t.dtype == torch.bfloat16 and t.stride(1) == 1, "skinny gemm: weight layout")
        n, k2 = w.shape
        _need(w_up is None or (w_up.shape == w.shape and w_up.stride(0) == w.stride(0)), "skinny gemm: shapes")
        ldw = w.stride(0)
    _need(k == k2, "skinny gemm: inner sizes")
    _need(m <= SKINNY_MAX_ROWS, f"skinny gemm: {m} rows")
    if add_to is not None:
        _need(add_to.dtype == torch.float32 and add_to.shape == (m, n), "skinny gemm: add_to")
        out, mode = add_to, 2
    else:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        mode = 0 if out_dtype == torch.bfloat16 else 1
        _need(out_dtype in (torch.bfloat16, torch.float32), "skinny gemm: output dtype")
    _check(
        lib,
        lib.hal_gemm_bf16_skinny(
            _ptr(x), k, _ptr(w), _ptr(w_up), ldw, _ptr(out), n, mode, m, n, k, _stream()
        ),
    )
    return out


def norm_folds(m: int, n: int, k: int, tiled: torch.Tensor | None) -> bool:
    """Whether a product of ``m`` rows against an ``[n, k]`` weight with a tiled copy
    takes an RMSNorm before or after it, or the rotation and the append, into itself: up
    to 16 rows always, 17 to 32 rows on matrices that the small-batch kernel still reads
    as fast as the library product does (not too large, rows not much longer than there
    are rows)."""
    if tiled is None or m <= 0 or k % 8:
        return False
    # (in captured graphs at 24 to 32 rows: o-proj 4096 x 4096 14-15 us against 18 for the
    # library product and a norm kernel; down 4096 x 14336 36-41 against 33-35, and
    # 3072 x 8192 22-25 against 21-22: two row tiles read the long rows of X twice as often)
    return m <= SKINNY_ROWS or (m <= FUSED_ROWS and n * k <= FUSED_MID_ELEMENTS and k <= 2 * n)


def gemm_bf16_skinny_norm(
    x: torch.Tensor | NormedRows,
    w_tiled: torch.Tensor,
    tiled_shape: tuple[int, int],
    w_up_tiled: torch.Tensor | None = None,
    next_norm: NextNorm | None = None,
):
    """``x @ w.T`` for at most 16 rows against a tiled bf16 weight, with the RMSNorm
    before it (``x`` is ``NormedRows``: the result is scaled per row; with ``w_up_tiled``
    the gated form) or after it (``next_norm``: the result is added into the float32
    stream ``next_norm.h`` and ``NormedRows`` for that norm come back) folded in."""
    lib = library.core_library()
    normed = x if isinstance(x, NormedRows) else None
    if normed is not None:
        x = normed.x
    _dev(x, w_tiled, w_up_tiled)
    m, k = x.shape
    n, k2 = tiled_shape
    _need(x.dtype == torch.bfloat16 and x.stride(1) == 1, "skinny gemm takes bf16 rows")
    _need(k == k2 and 0 < m <= FUSED_ROWS and k % 8 == 0, "skinny gemm with a folded norm: at most 32 rows, K in steps of 8")
    row_width = 16 * -(-m // 16)
    _need((normed is None) != (next_norm is None), "skinny gemm with a folded norm: the norm before or the one after")
    need = (-(-n // 16) * 16) * (-(-k // 32) * 32)
    for t in (w_tiled, w_up_tiled):
        if t is not None:
            _need(t.is_cuda and t.dtype == torch.bfloat16 and t.numel() == need and t.is_contiguous(), "skinny gemm: tiled weight")
    if next_norm is not None:
        h, nw = next_norm.h, next_norm.weight
        _need(w_up_tiled is None, "skinny gemm: the gated form cannot add into the stream")
        _need(h.dtype == torch.float32 and h.shape == (m, n) and h.is_contiguous(), "skinny gemm: residual stream")
        _need(nw.numel() == n and nw.dtype in (torch.float32, torch.bfloat16), "skinny gemm: norm weight")
        xw = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
        parts = torch.empty((-(-n // 16), row_width), dtype=torch.float32, device=x.device)
        _check(lib, lib.hal_gemm_bf16_skinny_norm(
            _ptr(x), x.stride(0), _ptr(w_tiled), None, 0, _ptr(h), n, m, n, k, None, 0, ctypes.c_float(0.0),
            _ptr(nw), dtype_code(nw.dtype), _ptr(xw), _ptr(parts), _stream()))
        return NormedRows(xw, parts, next_norm.eps, nw)
    _need(normed.ss_parts.shape[1] == row_width and normed.ss_parts.is_contiguous(), "skinny gemm: sums of squares")
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    _check(lib, lib.hal_gemm_bf16_skinny_norm(
        _ptr(x), x.stride(0), _ptr(w_tiled), _ptr(w_up_tiled), 0, _ptr(out), n, m, n, k,
        _ptr(normed.ss_parts), normed.ss_parts.shape[0], ctypes.c_float(normed.eps),
        None, 0, None, None, _stream()))
    return out


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype | None = None,
           tiled: torch.Tensor | None = None, next_norm: NextNorm | None = None):
    """``x @ w.T`` for a weight ``[out, in]``; ``tiled`` is ``tile_weight(w)`` if the
    model keeps that copy for small batches.  ``x`` may be ``NormedRows``; with
    ``next_norm`` the result may come back as ``NormedRows`` (already added into the
    stream) instead of a tensor.

    float32 weights: the true 32-bit kernel (activations are widened if needed).
    bf16 weights: the hand-written kernel where it is the faster one (``skinny_pays``:
    up to 16 rows); otherwise the library product that the reference itself uses for
    its linear layers (src/halite/transformers/infer/attention.py:21-24), except where
    float32 output is asked for and the library cannot give it, which the hand-written
    kernel does in passes of 64 rows.
    """
    if isinstance(x, NormedRows) or next_norm is not None:
        # ``next_norm``: where the product can, it adds its result into the stream itself
        # and returns ``NormedRows`` for that norm instead of the result
        m, k = x.shape
        if (w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and norm_folds(m, w.shape[0], k, tiled)
                and out_dtype in (None, torch.bfloat16)):
            if isinstance(x, NormedRows):
                return gemm_bf16_skinny_norm(x, tiled, tuple(w.shape))
            return gemm_bf16_skinny_norm(x, tiled, tuple(w.shape), next_norm=next_norm)
        if isinstance(x, NormedRows):
            x = x.materialize()
    out_dtype = out_dtype or x.dtype
    if w.dtype == torch.float32:
        y = gemm_f32(x if x.dtype == torch.float32 else x.float(), w)
        return y if out_dtype == torch.float32 else y.to(out_dtype)
    _need(w.dtype == torch.bfloat16, f"linear: weight dtype {w.dtype}")
    if x.dtype != torch.bfloat16:
        x = x.to(torch.bfloat16)
    m, k = x.shape
    skinny_ok = k % 8 == 0 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0
    if m <= SKINNY_ROWS and tiled is not None and k % 8 == 0:
        return gemm_bf16_skinny(x, tiled, out_dtype=out_dtype, tiled_shape=tuple(w.shape))
    if skinny_ok and skinny_pays(m, w.shape[0], k, False):
        return gemm_bf16_skinny(x, w, out_dtype=out_dtype)
    if out_dtype == torch.float32:
        global _MM_OUT_DTYPE
        if _MM_OUT_DTYPE is None:
            try:
                torch.mm(x[:1], w[:8].t(), out_dtype=torch.float32)
                _MM_OUT_DTYPE = True
            except (TypeError, RuntimeError):
                _MM_OUT_DTYPE = False
        if _MM_OUT_DTYPE:  # float32 accumulators written out unrounded
            return torch.mm(x, w.t(), out_dtype=torch.float32)
        if skinny_ok:
            out = torch.empty((m, w.shape[0]), dtype=torch.float32, device=x.device)
            for r0 in range(0, m, SKINNY_MAX_ROWS):
                out[r0 : r0 + SKINNY_MAX_ROWS] = gemm_bf16_skinny(
                    x[r0 : r0 + SKINNY_MAX_ROWS], w, out_dtype=torch.float32
                )
            return out
    y = torch.matmul(x, w.t())
    return y if out_dtype == torch.bfloat16 else y.to(out_dtype)
