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


@dataclass(frozen=True)
class ScoreRule:
    """What an attention does to its scores beside scaling them, and which keys a query
    sees beside the causal rule and a window.  ``chunk``: a query sees no key before the
    start of its own chunk of that many positions (counted from position 0 of the
    request).  ``bias``: float32 ``[heads, distances]`` on the device, added to the scaled
    score of the key ``n`` tokens back at ``[head, min(n, distances - 1)]``.  ``sink``: the
    softmax has one more term of score 0 that carries no value.  ``sigmoid``: no softmax: a
    visible key's weight is the sigmoid of its score (scaled, with the bias), and the weights
    are not normalised over the keys.  ``softcap`` > 0: the scaled score ``s`` becomes
    ``softcap * tanh(s / softcap)`` before the bias.  ``sink_values`` (with ``sink``): float32
    ``[heads]`` on the device, the score of the sink's term of every head instead of 0 (it is
    neither scaled nor capped)."""

    chunk: int = 0
    bias: torch.Tensor | None = None
    sink: bool = False
    # the same table times log2 e, for the kernel whose exponentials are to the base 2
    bias_log2: torch.Tensor | None = None
    sigmoid: bool = False
    softcap: float = 0.0
    sink_values: torch.Tensor | None = None
    # the same values times log2 e
    sink_values_log2: torch.Tensor | None = None

    def plain(self) -> bool:
        return (self.chunk == 0 and self.bias is None and not self.sink and not self.sigmoid
                and self.softcap == 0.0)

    def sink_checked(self, n_heads: int, log2: bool) -> torch.Tensor | None:
        """The sinks' values as a kernel takes them (None: every sink has the score 0)."""
        if self.sink_values is None:
            return None
        t = self.sink_values_log2 if log2 else self.sink_values
        if not self.sink or t is None or t.dtype != torch.float32 or t.shape != (n_heads,) or not t.is_contiguous():
            raise KernelError("sink values are float32 [heads] (and their multiples of log2 e), with sink=True")
        return t

    def weights_code(self) -> int:
        """The kernels' number for how a row's weights are made (``HAL_WEIGHTS_*``)."""
        if self.sigmoid and self.sink:
            raise KernelError("a sink belongs to a softmax; sigmoid weights have none")
        return 2 if self.sigmoid else (1 if self.sink else 0)


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


def embedding(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor | None = None, scale: float = 1.0):
    """``out[t] = table[ids[t]] * scale`` as float32."""
    lib = library.core_library()
    _dev(ids, table, out)
    _i32(ids, "ids")
    n, (vocab, d) = ids.numel(), table.shape
    if out is None:
        out = torch.empty((n, d), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (n, d), "embedding: bad output")
    _check(
        lib,
        lib.hal_embedding_scaled(_ptr(ids), _ptr(table), dtype_code(table.dtype), _ptr(out), n, d, vocab,
                                 ctypes.c_float(scale), _stream()),
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
    rule: ScoreRule | None = None,
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
    rule = rule or ScoreRule()
    bias = rule.bias
    if bias is not None:
        _dev(bias)
        _need(bias.dtype == torch.float32 and bias.dim() == 2 and bias.shape[0] == n_heads and bias.shape[1] > 0,
              "attention: the bias is float32 [heads, distances]")
    sinks = rule.sink_checked(n_heads, log2=False)
    _dev(sinks)
    _check(
        lib,
        lib.hal_attention_simple_ruled(
            _ptr(q), q_row_stride, _ptr(out), n_heads * head_dim, dtype_code(q.dtype),
            _ptr(positions), _ptr(token_seg), _ptr(block_table), block_table.shape[1],
            _ptr(k_pages), _ptr(v_pages), _ptr(part), n, n_heads, n_kv, head_dim, page_size, n_pages,
            ctypes.c_float(scale), window, rule.chunk, _ptr(bias), 0 if bias is None else bias.shape[1],
            rule.weights_code(), ctypes.c_float(rule.softcap), _ptr(sinks), max_kv_len, min_q_len, _stream(),
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
    relu_squared: bool = False,
):
    """``x @ w.T`` for at most 64 rows of bf16 ``x``; with ``w_up`` the gated form
    ``(x @ w_up.T) * silu(x @ w.T)``; ``add_to`` (float32) receives ``+=``;
    ``relu_squared``: the bf16 result is the square of relu of the product."""
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
    if relu_squared:
        _need(mode == 0 and w_up is None, "skinny gemm: the square of relu goes with a plain bf16 result")
        mode = 3
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


def linear_add(h: torch.Tensor, x: torch.Tensor, w: torch.Tensor, tiled: torch.Tensor | None = None) -> None:
    """``h += x @ w.T`` for the float32 stream ``h``: the product is float32 and the sum is
    made in float32; few bf16 rows do both in one kernel."""
    m, k = x.shape
    if (w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and m <= SKINNY_ROWS and tiled is not None and k % 8 == 0):
        gemm_bf16_skinny(x, tiled, add_to=h, tiled_shape=tuple(w.shape))
        return
    residual_add(h, linear(x, w, out_dtype=torch.float32, tiled=tiled))


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


# -- products in groups, and the kernels around a latent attention and a mixture of experts --

GROUP_TILE_ROWS = 128  # rows of a tile of the grouped product (what ``moe_sort`` counts tiles in)


def rmsnorm_exact(h: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
                  rows: torch.Tensor | None = None, second: torch.Tensor | None = None):
    """RMSNorm of the float32 stream ``h`` (only of ``rows`` if given) as ``x * rstd * w``
    in float32 with one rounding at the end; with ``second`` (another weight for the same
    rows) both results come back."""
    lib = library.core_library()
    _dev(h, weight, rows, second)
    _i32(rows, "rows")
    _need(h.dtype == torch.float32 and h.dim() == 2, "rmsnorm: the stream is float32 [T, d]")
    d = h.shape[1]
    _need(weight.shape == (d,) and (second is None or (second.shape == (d,) and second.dtype == weight.dtype)),
          "rmsnorm: weights of the stream's width and of one element type")
    n = h.shape[0] if rows is None else rows.numel()
    out1 = torch.empty((n, d), dtype=out_dtype, device=h.device)
    out2 = torch.empty((n, d), dtype=out_dtype, device=h.device) if second is not None else None
    _check(lib, lib.hal_norm_pair(_ptr(h), _ptr(rows), _ptr(weight), _ptr(second), dtype_code(weight.dtype),
                                  ctypes.c_float(eps), _ptr(out1), _ptr(out2), dtype_code(out_dtype), n, d, _stream()))
    return out1 if second is None else (out1, out2)


def latent_prep(a: torch.Tensor, q_col0: int, q_rank: int, kv_col0: int, kv_rank: int, rot: int, head_dim: int,
                w_q: torch.Tensor | None, w_kv: torch.Tensor, eps: float, qkv: torch.Tensor, k_col0: int):
    """From the float32 down projections ``a`` of a latent attention: the normed query
    latent ``[T, q_rank]`` (returned, of ``qkv``'s element type; None if ``q_rank`` is 0),
    and in the packed rows ``qkv`` the key row ``[rot | normed latent | 0]`` at column
    ``k_col0`` and the value row ``[0 | normed latent | 0]`` behind it, ``head_dim`` columns each."""
    lib = library.core_library()
    _dev(a, w_q, w_kv, qkv)
    n = a.shape[0]
    _need(a.dtype == torch.float32 and a.dim() == 2 and qkv.dim() == 2 and qkv.shape[0] == n, "latent_prep: rows")
    _need(w_kv.numel() == kv_rank and (q_rank == 0 or (w_q is not None and w_q.numel() == q_rank and w_q.dtype == w_kv.dtype)),
          "latent_prep: norm weights")
    _need(q_col0 + q_rank <= a.shape[1] and kv_col0 + kv_rank + rot <= a.shape[1] and head_dim >= rot + kv_rank
          and k_col0 + 2 * head_dim <= qkv.shape[1], "latent_prep: columns")
    cq = torch.empty((n, q_rank), dtype=qkv.dtype, device=a.device) if q_rank else None
    _check(lib, lib.hal_latent_prep(
        _ptr(a), a.shape[1], q_col0, q_rank, kv_col0, kv_rank, rot, head_dim, _ptr(w_q), _ptr(w_kv),
        dtype_code(w_kv.dtype), ctypes.c_float(eps), _ptr(cq), _ptr(qkv), qkv.shape[1], k_col0,
        dtype_code(qkv.dtype), n, _stream()))
    return cq


def head_cols(x: torch.Tensor, x_head: int, x0: int, y: torch.Tensor, y_head: int, y0: int, n: int,
              n_heads: int, zero_from: int = 0, n_zero: int = 0) -> None:
    """``y[t, h * y_head + y0 + j] = x[t, h * x_head + x0 + j]`` for ``j < n`` and every head,
    and zeros in the ``n_zero`` columns from ``h * y_head + zero_from``."""
    lib = library.core_library()
    _dev(x, y)
    _need(x.dim() == 2 and y.dim() == 2 and x.shape[0] == y.shape[0] and x.dtype == y.dtype, "head_cols: rows")
    _check(lib, lib.hal_head_cols(_ptr(x), x.shape[1], x_head, x0, _ptr(y), y.shape[1], y_head, y0, n,
                                  zero_from, n_zero, n_heads, dtype_code(x.dtype), x.shape[0], _stream()))


def scale_(x: torch.Tensor, s: float) -> torch.Tensor:
    """``x *= s`` in place (float32)."""
    lib = library.core_library()
    _dev(x)
    _need(x.dtype == torch.float32, "scale_: float32")
    if s != 1.0:
        _check(lib, lib.hal_scale_f32(_ptr(x), ctypes.c_longlong(x.numel()), ctypes.c_float(s), _stream()))
    return x


def grouped_gemm(
    x: torch.Tensor, w: torch.Tensor, y: torch.Tensor, *, n_rows: int,
    x_group_cols: int = 0, x_col0: int = 0, y_group_cols: int = 0, y_col0: int = 0,
    w_up: torch.Tensor | None = None, limit: float = 0.0, alpha: float = 0.0, up_shift: float = 1.0,
    group_offsets: torch.Tensor | None = None, tile_offsets: torch.Tensor | None = None,
    row_src: torch.Tensor | None = None, src_div: int = 1, row_dst: torch.Tensor | None = None,
    gate: torch.Tensor | None = None, add: bool = False, mfma: bool = True, relu_squared: bool = False,
    gate_per_group: bool = False,
) -> torch.Tensor:
    """``y_g = x_g @ w[g].T`` for every group ``g`` of ``w`` ``[G, N, K]`` in one launch
    (float32 accumulation).  Heads: every group has all ``n_rows`` rows; group ``g`` reads
    the ``K`` columns from ``g * x_group_cols + x_col0`` of ``x`` and writes the ``N``
    columns from ``g * y_group_cols + y_col0`` of ``y``; ``gate`` (float32, row-strided)
    multiplies the result by ``sigmoid(gate[t, g * y_group_cols + n])`` (``gate_per_group``: by
    ``sigmoid(gate[t, g])``, one number a group).  Experts:
    ``group_offsets`` / ``tile_offsets`` (from ``moe_sort``) cut a list of ``n_rows`` rows
    into the groups' slices; row ``i`` reads ``x[row_src[i] // src_div]`` and writes
    ``y[row_dst[i]]`` (``i`` without the arrays); with ``w_up`` the result is the clamped
    gated activation of the two products, ``g sigmoid(alpha g) (u + up_shift)`` with ``g`` and
    ``u`` held to ``limit`` (``inf``: not held); without it and with ``relu_squared`` the square of
    the product's positive part.  ``add``: added into a float32 ``y``."""
    lib = library.core_library()
    _dev(w, w_up, group_offsets, tile_offsets, row_src, row_dst)
    for t in (x, y, gate):
        _need(t is None or (t.is_cuda and t.dim() == 2 and t.stride(1) == 1), "grouped_gemm: rows on the GPU")
    _i32(group_offsets, "group_offsets"), _i32(tile_offsets, "tile_offsets"), _i32(row_src, "row_src"), _i32(row_dst, "row_dst")
    _need(w.dim() == 3 and w.dtype == x.dtype and (w_up is None or (w_up.shape == w.shape and w_up.dtype == w.dtype)),
          "grouped_gemm: weights [G, N, K] of the rows' element type")
    g, n, k = w.shape
    _need(not relu_squared or w_up is None, "grouped_gemm: the square of relu is for a product without a gate")
    _need(gate is None or gate.dtype == torch.float32, "grouped_gemm: a float32 gate")
    _need(not add or y.dtype == torch.float32, "grouped_gemm: only a float32 result is added into")
    if group_offsets is None:
        _need(x.shape[0] >= n_rows and y.shape[0] >= n_rows, "grouped_gemm: rows")
        _need((g - 1) * x_group_cols + x_col0 + k <= x.shape[1] and (g - 1) * y_group_cols + y_col0 + n <= y.shape[1],
              "grouped_gemm: columns outside the rows")
        _need(gate is None or (gate.shape[0] >= n_rows and
                               (g <= gate.shape[1] if gate_per_group else (g - 1) * y_group_cols + n <= gate.shape[1])),
              "grouped_gemm: gate")
    else:
        _need(group_offsets.numel() == g + 1 and tile_offsets is not None and tile_offsets.numel() == g + 1, "grouped_gemm: offsets")
        _need(x_group_cols == 0 and y_group_cols == 0 and x_col0 + k <= x.shape[1] and y_col0 + n <= y.shape[1], "grouped_gemm: columns")
        _need(row_src is None or row_src.numel() >= n_rows, "grouped_gemm: row_src")
        _need(row_dst is None or row_dst.numel() >= n_rows, "grouped_gemm: row_dst")
        _need(row_src is not None or x.shape[0] >= n_rows, "grouped_gemm: rows of x")
        _need(row_dst is not None or y.shape[0] >= n_rows, "grouped_gemm: rows of y")
        _need(gate is None, "grouped_gemm: the gate is for groups that share their rows")
    _check(lib, lib.hal_grouped_gemm(
        _ptr(x), x.stride(0), x_group_cols, x_col0, _ptr(w), _ptr(w_up), ctypes.c_longlong(n * k), k,
        dtype_code(x.dtype), _ptr(y), y.stride(0), y_group_cols, y_col0, dtype_code(y.dtype), 1 if add else 0,
        n_rows, n, k, g, _ptr(group_offsets), _ptr(tile_offsets), _ptr(row_src), src_div, _ptr(row_dst),
        _ptr(gate), 0 if gate is None else gate.stride(0), 1 if gate_per_group else 0, ctypes.c_float(limit),
        ctypes.c_float(up_shift), ctypes.c_float(alpha),
        1 if relu_squared else 0, 1 if mfma else 0, _stream()))
    return y


def moe_route(z: torch.Tensor, top: int, softmax: bool = False, normalize: bool = True, norm_eps: float = 0.0):
    """The ``top`` experts of every token from float32 router logits ``z`` ``[T, E]``: indices
    ``[T, top]`` int32 and weights ``[T, top]`` float32 (sigmoid scores, or the softmax over
    the experts; divided by their sum + ``norm_eps`` if ``normalize``)."""
    lib = library.core_library()
    _need(z.is_cuda and z.dtype == torch.float32 and z.dim() == 2 and z.stride(1) == 1,
          "moe_route: float32 logits [T, E] (a row-strided view is allowed)")
    t, e = z.shape
    idx = torch.empty((t, top), dtype=torch.int32, device=z.device)
    wgt = torch.empty((t, top), dtype=torch.float32, device=z.device)
    _check(lib, lib.hal_moe_route(_ptr(z), z.stride(0), e, top, 1 if softmax else 0, 1 if normalize else 0,
                                  ctypes.c_float(norm_eps), _ptr(idx), _ptr(wgt), t, _stream()))
    return idx, wgt


ROUTE_SORT_MAX_TOKENS = 16  # up to so many tokens (one a wave) one workgroup routes and sorts


def moe_route_sort(z: torch.Tensor, top: int, n_experts: int, softmax: bool = False, normalize: bool = True,
                   norm_eps: float = 0.0):
    """``moe_route`` and ``moe_sort`` in one launch: ``(idx, wgt, offsets, tile_offsets, sorted)``."""
    lib = library.core_library()
    _need(z.is_cuda and z.dtype == torch.float32 and z.dim() == 2 and z.stride(1) == 1 and z.shape[1] == n_experts,
          "moe_route_sort: float32 logits [T, E] (a row-strided view is allowed)")
    t = z.shape[0]
    idx = torch.empty((t, top), dtype=torch.int32, device=z.device)
    wgt = torch.empty((t, top), dtype=torch.float32, device=z.device)
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=z.device)
    tile_offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=z.device)
    order = torch.empty(max(t * top, 1), dtype=torch.int32, device=z.device)
    _check(lib, lib.hal_moe_route_sort(_ptr(z), z.stride(0), n_experts, top, 1 if softmax else 0, 1 if normalize else 0,
                                       ctypes.c_float(norm_eps), _ptr(idx), _ptr(wgt), t, GROUP_TILE_ROWS, _ptr(offsets),
                                       _ptr(tile_offsets), _ptr(order), _stream()))
    return idx, wgt, offsets, tile_offsets, order


def moe_sort(idx: torch.Tensor, n_experts: int):
    """The (token, choice) pairs of ``idx`` ``[T, top]`` sorted by expert on the device:
    ``offsets`` and ``tile_offsets`` ``[E + 1]`` and ``sorted`` ``[T * top]`` (pair numbers
    ``token * top + choice``), as ``grouped_gemm`` takes them."""
    lib = library.core_library()
    _dev(idx)
    _i32(idx, "idx")
    n = idx.numel()
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=idx.device)
    tile_offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=idx.device)
    order = torch.empty(max(n, 1), dtype=torch.int32, device=idx.device)
    _check(lib, lib.hal_moe_sort(_ptr(idx), n, n_experts, GROUP_TILE_ROWS, _ptr(offsets), _ptr(tile_offsets), _ptr(order), _stream()))
    return offsets, tile_offsets, order


def moe_combine(h: torch.Tensor, y: torch.Tensor, wgt: torch.Tensor, extra: torch.Tensor | None = None,
                extra_gate: torch.Tensor | None = None, overwrite: bool = False) -> None:
    """``h[t] += sum_j wgt[t, j] * y[t * top + j] (+ extra[t])`` (all float32); with
    ``extra_gate`` (float32 ``[T, 1]``, a row-strided view is allowed) ``extra[t]`` is
    multiplied by ``sigmoid(extra_gate[t])``.  ``overwrite``: ``h[t]`` becomes the sum (what it held is not read)."""
    lib = library.core_library()
    _dev(h, y, wgt, extra)
    t, top = wgt.shape
    _need(extra is None or (extra.dtype == torch.float32 and extra.shape == h.shape), "moe_combine: extra like h")
    _need(h.dtype == y.dtype == wgt.dtype == torch.float32 and h.shape[0] == t and y.shape == (t * top, h.shape[1]),
          "moe_combine: float32 h [T, d], y [T * top, d], weights [T, top]")
    if extra_gate is not None:
        _need(extra is not None and extra_gate.is_cuda and extra_gate.dtype == torch.float32
              and extra_gate.shape == (t, 1), "moe_combine: a float32 gate [T, 1] for the extra rows")
    _check(lib, lib.hal_moe_combine(_ptr(h), _ptr(y), _ptr(wgt), _ptr(extra), _ptr(extra_gate),
                                    0 if extra_gate is None else extra_gate.stride(0), top, h.shape[1], t,
                                    1 if overwrite else 0, _stream()))


def clamped_gate_mul(gate_up: torch.Tensor, limit: float, alpha: float, up_shift: float = 1.0) -> torch.Tensor:
    """``g * sigmoid(alpha * g) * (u + up_shift)`` with ``g = min(gate, limit)`` and
    ``u = clamp(up, -limit, limit)`` of rows ``[gate | up]``."""
    lib = library.core_library()
    _dev(gate_up)
    n, two_f = gate_up.shape
    _need(two_f % 2 == 0, "clamped_gate_mul: odd row length")
    out = torch.empty((n, two_f // 2), dtype=gate_up.dtype, device=gate_up.device)
    _check(lib, lib.hal_clamped_gate_mul(_ptr(gate_up), _ptr(out), dtype_code(gate_up.dtype), n, two_f // 2,
                                         ctypes.c_float(limit), ctypes.c_float(alpha), ctypes.c_float(up_shift), _stream()))
    return out


# -- rows of the stream and of projections; mixers with a carried state -----------------------


def cast_rows(h: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """The float32 rows ``h`` rounded to ``dtype`` (``h`` itself if that is float32)."""
    if dtype == torch.float32:
        return h
    lib = library.core_library()
    _dev(h)
    _need(h.dtype == torch.float32, "cast_rows: float32 rows")
    out = torch.empty(h.shape, dtype=dtype, device=h.device)
    _check(lib, lib.hal_cast_rows(_ptr(h), _ptr(out), dtype_code(dtype), ctypes.c_longlong(h.numel()), _stream()))
    return out


def post_norm_add(h: torch.Tensor, a: torch.Tensor, weight: torch.Tensor, eps: float,
                  cast_to: torch.dtype | None = None, scale: float = 1.0, second: torch.Tensor | None = None,
                  second_scale: float = 0.0):
    """``h += x * rsqrt(mean(x^2) + eps) * weight`` row by row in float32 with
    ``x = scale * a`` (``+ second_scale * second``: the sum of two parts' results); ``h``,
    ``a`` and ``second`` float32 ``[T, d]``; with ``cast_to`` the new rows rounded to that
    type come back."""
    lib = library.core_library()
    _dev(h, a, weight, second)
    _need(h.dtype == torch.float32 and a.dtype == torch.float32 and h.dim() == 2 and a.shape == h.shape,
          "post_norm_add: float32 rows of one shape")
    _need(second is None or (second.dtype == torch.float32 and second.shape == h.shape), "post_norm_add: the second term")
    _need(weight.shape == (h.shape[1],), "post_norm_add: weight of the rows' width")
    cast = None
    if cast_to is not None and cast_to != torch.float32:
        cast = torch.empty(h.shape, dtype=cast_to, device=h.device)
    _check(lib, lib.hal_post_norm_add(_ptr(h), _ptr(a), _ptr(second), ctypes.c_float(scale), ctypes.c_float(second_scale),
                                      _ptr(weight), dtype_code(weight.dtype), ctypes.c_float(eps),
                                      _ptr(cast), dtype_code(cast_to or torch.float32), h.shape[0], h.shape[1], _stream()))
    return h if cast is None else cast


def relu_squared(x: torch.Tensor) -> torch.Tensor:
    lib = library.core_library()
    _dev(x)
    out = torch.empty_like(x)
    _check(lib, lib.hal_relu_squared(_ptr(x), _ptr(out), dtype_code(x.dtype), ctypes.c_longlong(x.numel()), _stream()))
    return out


def scaled_sum_(y: torch.Tensor, alpha: float, x: torch.Tensor, beta: float) -> torch.Tensor:
    """``y = alpha * y + beta * x`` in place (float32)."""
    lib = library.core_library()
    _dev(y, x)
    _need(y.dtype == torch.float32 and x.dtype == torch.float32 and x.shape == y.shape, "scaled_sum_: float32 of one shape")
    _check(lib, lib.hal_scaled_sum_f32(_ptr(y), ctypes.c_float(alpha), _ptr(x), ctypes.c_float(beta),
                                       ctypes.c_longlong(y.numel()), _stream()))
    return y


def _rows_f32(t: torch.Tensor, cols: int, what: str):
    _need(t.is_cuda and t.dtype == torch.float32 and t.dim() == 2 and t.stride(1) == 1 and t.shape[1] == cols,
          f"{what}: float32 rows of {cols} columns on the GPU")


def qk_norm_pack(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor | None, w_q: torch.Tensor, w_k: torch.Tensor,
                 eps: float, n_heads: int, n_kv_heads: int, qk_dim: int, v_dim: int, head_dim: int,
                 out_dtype: torch.dtype, positions: torch.Tensor | None = None, temp_coef: float = 0.0,
                 temp_every: int = 0, token_seg: torch.Tensor | None = None, block_table: torch.Tensor | None = None,
                 k_pages: torch.Tensor | None = None, v_pages: torch.Tensor | None = None, page_size: int = 0,
                 tiled: bool = False) -> torch.Tensor:
    """From float32 projections (row-strided views allowed): ``q`` and ``k`` each divided by
    the root mean square of their whole row (all heads at once) and multiplied by their
    weights, ``q`` further by ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)`` at
    position ``p`` if ``temp_every`` > 0; the packed rows ``[q heads | k heads | v heads]``
    of ``head_dim`` entries a head (zero beyond ``qk_dim`` / ``v_dim``) come back.  ``v``
    None: the values are the keys as they were projected.  With ``k_pages`` and ``v_pages``
    keys and values are appended to the pages as well, as ``rope_append`` does it (for an
    attention that does not rotate)."""
    lib = library.core_library()
    n = q.shape[0]
    _rows_f32(q, n_heads * qk_dim, "qk_norm_pack q"), _rows_f32(k, n_kv_heads * qk_dim, "qk_norm_pack k")
    if v is not None:
        _rows_f32(v, n_kv_heads * v_dim, "qk_norm_pack v")
    _dev(w_q, w_k, positions)
    _i32(positions, "positions")
    _need(w_q.numel() == n_heads * qk_dim and w_k.numel() == n_kv_heads * qk_dim and w_q.dtype == w_k.dtype,
          "qk_norm_pack: norm weights")
    _need(head_dim >= max(qk_dim, v_dim) and (v is not None or v_dim == qk_dim), "qk_norm_pack: head sizes")
    _need(temp_every == 0 or (positions is not None and positions.numel() == n), "qk_norm_pack: positions")
    out = torch.empty((n, (n_heads + 2 * n_kv_heads) * head_dim), dtype=out_dtype, device=q.device)
    n_pages = 0
    if k_pages is not None:
        _dev(token_seg, block_table, k_pages, v_pages)
        _i32(token_seg, "token_seg"), _i32(block_table, "block_table")
        n_pages = k_pages.shape[0]
        _need(v_pages is not None and k_pages.dtype == out_dtype and v_pages.dtype == out_dtype
              and k_pages.shape == (n_pages, n_kv_heads, page_size, head_dim)
              and v_pages.shape == (n_pages, n_kv_heads, head_dim, page_size), "qk_norm_pack: page shapes")
        _need(positions is not None and positions.numel() == n and token_seg is not None and token_seg.numel() == n
              and block_table is not None and block_table.dim() == 2, "qk_norm_pack: the step's arrays")
    _check(lib, lib.hal_qk_norm_pack(
        _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), 0 if v is None else v.stride(0), _ptr(w_q), _ptr(w_k),
        dtype_code(w_q.dtype), ctypes.c_float(eps), _ptr(positions), ctypes.c_float(temp_coef), temp_every,
        _ptr(out), out.shape[1], dtype_code(out_dtype), n, n_heads, n_kv_heads, qk_dim, v_dim, head_dim,
        _ptr(token_seg), _ptr(block_table), 0 if block_table is None else block_table.shape[1],
        _ptr(k_pages), _ptr(v_pages), page_size, n_pages, 1 if tiled else 0, _stream()))
    return out


def short_conv(u: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, state: torch.Tensor,
               token_seg: torch.Tensor, seg_q_start: torch.Tensor, token_slot: torch.Tensor,
               out_dtype: torch.dtype, silu: bool = False, in_bias: torch.Tensor | None = None) -> torch.Tensor:
    """The causal convolution over time ``y[t, c] = act(bias[c] + sum_j weight[c, j] *
    u[t - taps + 1 + j, c])`` on the step's flat batch: ``u`` float32 ``[T, C]`` (a
    row-strided view is allowed), ``state`` float32 ``[slots, taps - 1, C]`` the inputs of
    every request before this step (zeros for a new one; not changed here).  ``in_bias``
    ``[C]``: added to every input of the step where it is read (the bias of the projection that
    made ``u``; the state rows hold inputs with it, the zeros before a request's start are zeros)."""
    lib = library.core_library()
    c, taps = weight.shape
    _rows_f32(u, c, "short_conv")
    _dev(weight, bias, state, token_seg, seg_q_start, token_slot, in_bias)
    _need(in_bias is None or in_bias.shape == (c,), "short_conv: in_bias")
    _i32(token_seg, "token_seg"), _i32(seg_q_start, "seg_q_start"), _i32(token_slot, "token_slot")
    n = u.shape[0]
    _need(state.dtype == torch.float32 and state.dim() == 3 and state.shape[1:] == (taps - 1, c), "short_conv: state rows")
    _need(bias is None or (bias.shape == (c,) and bias.dtype == weight.dtype), "short_conv: bias")
    _need(token_seg.numel() == n and token_slot.numel() == n, "short_conv: one segment and slot a token")
    y = torch.empty((n, c), dtype=out_dtype, device=u.device)
    _check(lib, lib.hal_short_conv(
        _ptr(u), u.stride(0), _ptr(weight), _ptr(bias), dtype_code(weight.dtype), _ptr(in_bias),
        F32 if in_bias is None else dtype_code(in_bias.dtype), taps, _ptr(state), _ptr(token_seg),
        _ptr(seg_q_start), _ptr(token_slot), _ptr(y), c, dtype_code(out_dtype), 1 if silu else 0, n, c, _stream()))
    return y


def short_conv_through(u: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, state: torch.Tensor,
                       ctx, out_dtype: torch.dtype, silu: bool = False, in_bias: torch.Tensor | None = None) -> torch.Tensor:
    """``short_conv`` and ``short_conv_carry`` for the step ``ctx``: the convolution's result,
    and the state left as the next step finds it.  A step in which every request brings
    one token takes one kernel for both."""
    c, taps = weight.shape
    n = u.shape[0]
    if taps == 1:
        return short_conv(u, weight, bias, state, ctx.token_seg, ctx.seg_q_start, ctx.token_slot, out_dtype, silu, in_bias)
    if n == ctx.n_segs:
        lib = library.core_library()
        _rows_f32(u, c, "short_conv")
        _dev(weight, bias, state, in_bias)
        _need(in_bias is None or in_bias.shape == (c,), "short_conv: in_bias")
        slot = ctx.token_slot
        _dev(slot)
        _i32(slot, "token_slot")
        _need(state.dtype == torch.float32 and state.dim() == 3 and state.shape[1:] == (taps - 1, c), "short_conv: state rows")
        _need(bias is None or (bias.shape == (c,) and bias.dtype == weight.dtype), "short_conv: bias")
        _need(slot.numel() == n, "short_conv: one slot a token")
        y = torch.empty((n, c), dtype=out_dtype, device=u.device)
        _check(lib, lib.hal_short_conv_step(
            _ptr(u), u.stride(0), _ptr(weight), _ptr(bias), dtype_code(weight.dtype), _ptr(in_bias),
            F32 if in_bias is None else dtype_code(in_bias.dtype), taps, _ptr(state), _ptr(slot),
            _ptr(y), c, dtype_code(out_dtype), 1 if silu else 0, n, c, _stream()))
        return y
    y = short_conv(u, weight, bias, state, ctx.token_seg, ctx.seg_q_start, ctx.token_slot, out_dtype, silu, in_bias)
    short_conv_carry(u, state, ctx.seg_q_start, ctx.seg_q_len, ctx.token_slot, in_bias)
    return y


def short_conv_carry(u: torch.Tensor, state: torch.Tensor, seg_q_start: torch.Tensor, seg_q_len: torch.Tensor,
                     token_slot: torch.Tensor, in_bias: torch.Tensor | None = None) -> None:
    """After ``short_conv``: every request's state becomes the last ``taps - 1`` of (its
    state, then its inputs of this step)."""
    lib = library.core_library()
    c = state.shape[2]
    _rows_f32(u, c, "short_conv_carry")
    _dev(state, seg_q_start, seg_q_len, token_slot, in_bias)
    _need(state.dtype == torch.float32 and state.dim() == 3, "short_conv_carry: state rows")
    _need(seg_q_start.numel() == seg_q_len.numel(), "short_conv_carry: segment arrays")
    _check(lib, lib.hal_short_conv_carry(_ptr(u), u.stride(0), _ptr(in_bias),
                                         F32 if in_bias is None else dtype_code(in_bias.dtype),
                                         _ptr(state), state.shape[1] + 1, _ptr(seg_q_start),
                                         _ptr(seg_q_len), _ptr(token_slot), seg_q_start.numel(), c, _stream()))


def ssd_scan(xbc: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor,
             d_skip: torch.Tensor, state: torch.Tensor, seg_q_start: torch.Tensor, seg_q_len: torch.Tensor,
             token_slot: torch.Tensor, groups: int, chunks: torch.Tensor | None = None,
             seg_chunks: torch.Tensor | None = None, fixed_decay: torch.Tensor | None = None,
             in_silu: bool = False) -> torch.Tensor:
    """The state-space recurrence over every request's tokens of the step.  ``xbc``
    ``[T, heads * P + 2 * groups * N]``: x, then B and C; ``dt_raw`` float32 ``[T, heads]``
    (a row-strided view is allowed); ``state`` float32 ``[slots, heads, N, P]``, read and
    left as the step's last state.  Returns float32 ``[T, heads * P]``.  ``chunks`` int32
    ``[n, 4]`` (first token, tokens, segment, 0) and ``seg_chunks`` ``[segments, 2]`` (first
    chunk, chunks): the segments cut into chunks that are walked side by side (what long
    prompts need to fill the chip); without them a wave walks a whole segment.
    ``fixed_decay`` float32 ``[heads]``: one constant decay a head, every step size 1 and nothing
    added for the token itself (``dt_raw``, ``dt_bias``, ``a_log`` and ``d_skip`` are None):
    ``S <- decay S + B x^T``, ``y = S^T C``.  ``in_silu``: x, B and C are SiLU of what ``xbc``
    holds.  ``xbc`` may be a row-strided view."""
    lib = library.core_library()
    _dev(dt_bias, a_log, d_skip, state, seg_q_start, seg_q_len, token_slot, fixed_decay)
    _need(xbc.is_cuda and xbc.dim() == 2 and xbc.stride(1) == 1, "ssd_scan: rows on the GPU")
    _, heads, n_state, p = state.shape
    n = xbc.shape[0]
    _need(state.dtype == torch.float32 and xbc.dim() == 2 and xbc.shape[1] == heads * p + 2 * groups * n_state,
          "ssd_scan: rows of x, B and C")
    if fixed_decay is not None:
        _need(fixed_decay.dtype == torch.float32 and fixed_decay.shape == (heads,) and dt_raw is None and dt_bias is None
              and a_log is None and d_skip is None, "ssd_scan: fixed decays are float32 [heads] and come alone")
    else:
        _need(dt_raw.is_cuda and dt_raw.dtype == torch.float32 and dt_raw.shape == (n, heads) and dt_raw.stride(1) == 1,
              "ssd_scan: float32 step sizes [T, heads]")
        _need(dt_bias.numel() == heads and a_log.numel() == heads and d_skip.numel() == heads
              and dt_bias.dtype == a_log.dtype == d_skip.dtype, "ssd_scan: one bias, rate and skip a head, of one type")
    y = torch.empty((n, heads * p), dtype=torch.float32, device=xbc.device)
    sums = decays = None
    n_chunks = 0
    if chunks is not None:
        _dev(chunks, seg_chunks)
        _i32(chunks, "chunks"), _i32(seg_chunks, "seg_chunks")
        _need(chunks.dim() == 2 and chunks.shape[1] == 4 and seg_chunks is not None
              and seg_chunks.shape == (seg_q_start.numel(), 2), "ssd_scan: chunk arrays")
        n_chunks = chunks.shape[0]
        sums = torch.empty((n_chunks, heads, n_state, p), dtype=torch.float32, device=xbc.device)
        decays = torch.empty((n_chunks, heads), dtype=torch.float32, device=xbc.device)
    _check(lib, lib.hal_ssd_scan(
        _ptr(xbc), xbc.stride(0), dtype_code(xbc.dtype), _ptr(dt_raw), 0 if dt_raw is None else dt_raw.stride(0),
        _ptr(dt_bias), _ptr(a_log), _ptr(d_skip), F32 if a_log is None else dtype_code(a_log.dtype), _ptr(state), _ptr(seg_q_start), _ptr(seg_q_len), _ptr(token_slot),
        _ptr(y), seg_q_start.numel(), heads, p, n_state, groups, _ptr(chunks), _ptr(seg_chunks), n_chunks,
        _ptr(sums), _ptr(decays), _ptr(fixed_decay), 1 if in_silu else 0, _stream()))
    return y


def gated_part_norm(y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, eps: float, parts: int,
                    out_dtype: torch.dtype) -> torch.Tensor:
    """``(y * silu(z))`` with every one of ``parts`` equal parts of a row divided by its
    own root mean square, times ``weight`` (``y`` float32 ``[T, n]``, ``z`` float32, a
    row-strided view is allowed)."""
    lib = library.core_library()
    _dev(y, weight)
    n, inner = y.shape
    _rows_f32(z, inner, "gated_part_norm z")
    _need(y.dtype == torch.float32 and weight.numel() == inner and inner % parts == 0, "gated_part_norm: sizes")
    out = torch.empty((n, inner), dtype=out_dtype, device=y.device)
    _check(lib, lib.hal_gated_part_norm(_ptr(y), _ptr(z), z.stride(0), _ptr(weight), dtype_code(weight.dtype),
                                        ctypes.c_float(eps), _ptr(out), dtype_code(out_dtype), n, inner, parts, _stream()))
    return out


# -- the generalized delta rule; copies of the stream; per-head norms and gates -------------------


def delta_rule(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a_raw: torch.Tensor, x1: torch.Tensor,
               w2: torch.Tensor, w0: torch.Tensor, a_bias: torch.Tensor, state: torch.Tensor,
               seg_q_start: torch.Tensor, seg_q_len: torch.Tensor, token_slot: torch.Tensor,
               decay_rate: float, unit_eps: float) -> torch.Tensor:
    """The generalized delta rule over every request's tokens of the step: per head
    ``S <- diag(w) S - (a * u)(u^T S) + k v^T``, ``o = S^T r`` with ``w = exp(-decay_rate *
    sigmoid(w0 + W2 tanh(x1)))``, ``a = sigmoid(a_raw + a_bias)`` and the unit key ``u = k /
    sqrt(sum(k^2) + unit_eps)``.  ``r``, ``k``, ``v``, ``a_raw``: float32 ``[T, heads * dim]``
    (row-strided views allowed); ``x1`` float32 ``[T, rank]``; ``state`` float32 ``[slots,
    heads, dim, dim]`` (key channel, value channel), read and left as the step's last state.
    Returns float32 ``[T, heads * dim]``."""
    lib = library.core_library()
    _, heads, d, d2 = state.shape
    n, inner = r.shape[0], heads * d
    for t, what in ((r, "r"), (k, "k"), (v, "v"), (a_raw, "a")):
        _rows_f32(t, inner, f"delta_rule {what}")
        _need(t.shape[0] == n, "delta_rule: one row a token")
    lora = x1.shape[1]
    _rows_f32(x1, lora, "delta_rule x1")
    _dev(w2, w0, a_bias, state, seg_q_start, seg_q_len, token_slot)
    _i32(seg_q_start, "seg_q_start"), _i32(seg_q_len, "seg_q_len"), _i32(token_slot, "token_slot")
    _need(state.dtype == torch.float32 and d == d2, "delta_rule: a float32 state [slots, heads, dim, dim]")
    _need(w2.shape == (inner, lora) and w0.numel() == inner and a_bias.numel() == inner
          and w2.dtype == w0.dtype == a_bias.dtype, "delta_rule: w2 [heads * dim, rank], w0 and a_bias [heads * dim] of one type")
    _need(token_slot.numel() == n and seg_q_start.numel() == seg_q_len.numel(), "delta_rule: the step's arrays")
    dp = 16 if d <= 16 else 32 if d <= 32 else 64 if d <= 64 else 128 if d <= 128 else 256
    pre = torch.empty((n, heads, 5, dp), dtype=torch.float32, device=r.device)
    o = torch.empty((n, inner), dtype=torch.float32, device=r.device)
    _check(lib, lib.hal_delta_rule(
        _ptr(r), r.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _ptr(a_raw), a_raw.stride(0),
        _ptr(x1), x1.stride(0), _ptr(w2), _ptr(w0), _ptr(a_bias), dtype_code(w2.dtype), lora,
        ctypes.c_float(decay_rate), ctypes.c_float(unit_eps), _ptr(pre), _ptr(state), _ptr(seg_q_start),
        _ptr(seg_q_len), _ptr(token_slot), _ptr(o), n, seg_q_start.numel(), heads, d, _stream()))
    return o


def head_norm_gate(y: torch.Tensor, z: torch.Tensor | None, weight: torch.Tensor | None, eps: float, heads: int,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """Every head of the float32 rows ``y`` ``[T, heads * dim]`` divided by its own root mean
    square, times ``weight`` (of the row's length) and ``sigmoid(z)`` (float32, a row-strided
    view is allowed)."""
    lib = library.core_library()
    _dev(y, weight)
    n, inner = y.shape
    _need(y.dtype == torch.float32 and inner % heads == 0, "head_norm_gate: float32 rows of whole heads")
    if z is not None:
        _rows_f32(z, inner, "head_norm_gate z")
    _need(weight is None or weight.numel() == inner, "head_norm_gate: a weight of the row's length")
    out = torch.empty((n, inner), dtype=out_dtype, device=y.device)
    _check(lib, lib.hal_head_norm_gate(_ptr(y), _ptr(z), 0 if z is None else z.stride(0), _ptr(weight),
                                       dtype_code(weight.dtype) if weight is not None else F32, ctypes.c_float(eps),
                                       _ptr(out), dtype_code(out_dtype), n, heads, inner // heads, _stream()))
    return out


def streams_step(x: torch.Tensor, *, y: torch.Tensor | None = None, mix: torch.Tensor | None = None,
                 out: torch.Tensor | None = None, mult: float = 1.0, read: bool = False,
                 inw: torch.Tensor | None = None, norm_weight: torch.Tensor | None = None, offset: float = 0.0,
                 eps: float = 0.0, dtype: torch.dtype = torch.float32, rows: torch.Tensor | None = None):
    """One pass over the copies ``x`` (float32 ``[S, T, W]``) of the residual stream.  With
    ``y`` (float32 ``[T, W]``) every copy is made anew from the old ones, ``x_t <- sum_s
    mix[s, t] x_s + mult * out[t] * y``.  With ``read`` the row ``u = sum_s inw[s] x_s``
    (``inw`` None: the plain sum) of the new copies comes back, as it is (float32) or, with
    ``norm_weight``, as ``u / sqrt(mean(u^2) + eps) * (offset + norm_weight)`` in ``dtype``;
    ``rows`` (only without ``y``): of those rows alone."""
    lib = library.core_library()
    _dev(x, y, mix, out, inw, norm_weight, rows)
    _i32(rows, "rows")
    _need(x.dtype == torch.float32 and x.dim() == 3, "streams_step: float32 copies [S, T, W]")
    s, t, w = x.shape
    _need(y is None or (y.dtype == torch.float32 and y.shape == (t, w) and mix is not None and out is not None
                        and mix.shape == (s, s) and out.numel() == s and mix.dtype == out.dtype and rows is None),
          "streams_step: an update takes float32 y [T, W], mix [S, S] and out [S] of one type, and all rows")
    _need(inw is None or (inw.numel() == s and (mix is None or inw.dtype == mix.dtype)), "streams_step: inw [S]")
    _need(norm_weight is None or norm_weight.numel() == w, "streams_step: a norm weight of the rows' width")
    c_dtype = mix.dtype if mix is not None else (inw.dtype if inw is not None else torch.float32)
    n = t if rows is None else rows.numel()
    result = None
    if read:
        result = torch.empty((n, w), dtype=dtype if norm_weight is not None else torch.float32, device=x.device)
    _check(lib, lib.hal_streams_step(
        _ptr(x), ctypes.c_longlong(t * w), s, _ptr(y), _ptr(mix), _ptr(out), ctypes.c_float(mult), _ptr(inw),
        dtype_code(c_dtype), 1 if read else 0, _ptr(norm_weight),
        dtype_code(norm_weight.dtype) if norm_weight is not None else F32, ctypes.c_float(offset), ctypes.c_float(eps),
        _ptr(result), dtype_code(result.dtype) if result is not None else F32, _ptr(rows), n, w, _stream()))
    return result


def head_norm_pack(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, eps: float, n_heads: int, n_kv_heads: int,
                   qk_dim: int, v_dim: int, head_dim: int, out_dtype: torch.dtype,
                   positions: torch.Tensor | None = None, token_seg: torch.Tensor | None = None,
                   block_table: torch.Tensor | None = None, k_pages: torch.Tensor | None = None,
                   v_pages: torch.Tensor | None = None, page_size: int = 0, tiled: bool = False,
                   w_q: torch.Tensor | None = None, w_k: torch.Tensor | None = None, norm_v: bool = True,
                   v_other: torch.Tensor | None = None, v_mix: float = 0.0) -> torch.Tensor:
    """From float32 projections (row-strided views allowed): every head of ``q``, ``k`` and
    (with ``norm_v``) ``v`` divided by its own root mean square; the packed rows ``[q heads | k
    heads | v heads]`` of ``head_dim`` entries a head (zero beyond ``qk_dim`` / ``v_dim``) come
    back.  ``w_q`` / ``w_k`` ``[qk_dim]``: a weight that multiplies every normed head of q / k.
    ``v_other`` (float32 rows like ``v``): the values become ``(1 - v_mix) v + v_mix v_other``.
    With ``k_pages`` and ``v_pages`` keys and values are appended to the pages as well."""
    lib = library.core_library()
    _dev(w_q, w_k)
    _need((w_q is None) == (w_k is None) and (w_q is None or (w_q.shape == (qk_dim,) and w_k.shape == (qk_dim,)
                                                             and w_q.dtype == w_k.dtype)),
          "head_norm_pack: weights [qk_dim] of one type for q and k, or none")
    if v_other is not None:
        _rows_f32(v_other, n_kv_heads * v_dim, "head_norm_pack v_other")
        _need(v_other.shape[0] == q.shape[0], "head_norm_pack: one row of other values a token")
    n = q.shape[0]
    _rows_f32(q, n_heads * qk_dim, "head_norm_pack q"), _rows_f32(k, n_kv_heads * qk_dim, "head_norm_pack k")
    _rows_f32(v, n_kv_heads * v_dim, "head_norm_pack v")
    _need(head_dim >= max(qk_dim, v_dim), "head_norm_pack: head sizes")
    out = torch.empty((n, (n_heads + 2 * n_kv_heads) * head_dim), dtype=out_dtype, device=q.device)
    n_pages = 0
    if k_pages is not None:
        _dev(positions, token_seg, block_table, k_pages, v_pages)
        _i32(positions, "positions"), _i32(token_seg, "token_seg"), _i32(block_table, "block_table")
        n_pages = k_pages.shape[0]
        _need(v_pages is not None and k_pages.dtype == out_dtype and v_pages.dtype == out_dtype
              and k_pages.shape == (n_pages, n_kv_heads, page_size, head_dim)
              and v_pages.shape == (n_pages, n_kv_heads, head_dim, page_size), "head_norm_pack: page shapes")
        _need(positions is not None and positions.numel() == n and token_seg is not None and token_seg.numel() == n
              and block_table is not None and block_table.dim() == 2, "head_norm_pack: the step's arrays")
    _check(lib, lib.hal_head_norm_pack(
        _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), ctypes.c_float(eps),
        _ptr(w_q), _ptr(w_k), dtype_code(w_q.dtype) if w_q is not None else F32, 1 if norm_v else 0,
        _ptr(v_other), 0 if v_other is None else v_other.stride(0), ctypes.c_float(v_mix), _ptr(positions),
        _ptr(out), out.shape[1], dtype_code(out_dtype), n, n_heads, n_kv_heads, qk_dim, v_dim, head_dim,
        _ptr(token_seg), _ptr(block_table), 0 if block_table is None else block_table.shape[1],
        _ptr(k_pages), _ptr(v_pages), page_size, n_pages, 1 if tiled else 0, _stream()))
    return out


def head_gate_cols(x: torch.Tensor, x_head: int, gate: torch.Tensor, n: int, n_heads: int) -> torch.Tensor:
    """``y[t, h * n + j] = x[t, h * x_head + j] * sigmoid(gate[t, h])`` for ``j < n``: every
    head's first ``n`` entries times a number of the head's own (``gate`` float32, a
    row-strided view is allowed)."""
    lib = library.core_library()
    _dev(x)
    _need(x.dim() == 2 and x.shape[1] >= n_heads * x_head and x_head >= n, "head_gate_cols: rows of padded heads")
    _rows_f32(gate, n_heads, "head_gate_cols gate")
    _need(gate.shape[0] == x.shape[0], "head_gate_cols: one gate row a token")
    y = torch.empty((x.shape[0], n_heads * n), dtype=x.dtype, device=x.device)
    _check(lib, lib.hal_head_gate_cols(_ptr(x), x.shape[1], x_head, _ptr(gate), gate.stride(0), _ptr(y), n, n_heads,
                                       dtype_code(x.dtype), x.shape[0], _stream()))
    return y


# -- small passes over float32 rows of projections ----------------------------------------------


def bias_rows_(a: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """``a[t, c] += bias[c]`` in place on float32 rows (a row-strided view is allowed)."""
    lib = library.core_library()
    _dev(bias)
    _rows_f32(a, bias.numel(), "bias_rows_")
    _check(lib, lib.hal_bias_rows(_ptr(a), a.stride(0), _ptr(bias), dtype_code(bias.dtype), a.shape[0], a.shape[1], _stream()))
    return a


def silu_rows(a: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """``silu(a)`` of float32 rows (a row-strided view is allowed), rounded to ``out_dtype``."""
    lib = library.core_library()
    _rows_f32(a, a.shape[1], "silu_rows")
    out = torch.empty(a.shape, dtype=out_dtype, device=a.device)
    _check(lib, lib.hal_silu_rows(_ptr(a), a.stride(0), _ptr(out), dtype_code(out_dtype), a.shape[0], a.shape[1], _stream()))
    return out


def token_gate(g: torch.Tensor, table: torch.Tensor, col0: int, tokens: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """``gelu_tanh(g[t, j]) * table[tokens[t], col0 + j]`` for float32 rows ``g`` ``[T, dim]``
    and a table ``[vocab, columns]``; a token outside the table gives a NaN row."""
    lib = library.core_library()
    _dev(table, tokens)
    _i32(tokens, "tokens")
    n, dim = g.shape
    _rows_f32(g, dim, "token_gate")
    _need(table.dim() == 2 and 0 <= col0 and col0 + dim <= table.shape[1] and tokens.numel() == n, "token_gate: sizes")
    out = torch.empty((n, dim), dtype=out_dtype, device=g.device)
    _check(lib, lib.hal_token_gate(_ptr(g), g.stride(0), _ptr(table), dtype_code(table.dtype), table.shape[1], col0,
                                   _ptr(tokens), table.shape[0], _ptr(out), dtype_code(out_dtype), n, dim, _stream()))
    return out
