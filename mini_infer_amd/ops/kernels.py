"""Thin wrappers that hand torch tensors to the HIP entry points.

Each wrapper checks device, dtype and layout on the host, passes raw pointers and
the current HIP stream, and raises with the library's message when a kernel
refuses a size.  There is no CPU path: a CPU tensor is an error.
"""

from __future__ import annotations

import dataclasses
import math

import torch

from mini_infer_amd.exceptions import KernelShapeError
from mini_infer_amd.ops import library

F32, BF16 = 0, 1


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelShapeError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}")


def _need_cuda(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "mini_infer_amd kernels run on the GPU only (there is no CPU fallback); "
                f"got a tensor on {t.device}"
            )


def _need_contiguous(name: str, t: torch.Tensor | None) -> None:
    if t is not None and not t.is_contiguous():
        raise KernelShapeError(f"{name} must be contiguous, got strides {t.stride()}")


def _need_int32(name: str, t: torch.Tensor | None) -> None:
    if t is not None and t.dtype != torch.int32:
        raise KernelShapeError(f"{name} must be int32, got {t.dtype}")


def _check_v_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, v_transposed: bool, v_dim: int | None = None) -> None:
    pages, heads, page_size, head_dim = k_pages.shape
    head_dim = head_dim if v_dim is None else v_dim  # (value rows of a width of their own)
    expected = (pages, heads, head_dim, page_size) if v_transposed else (pages, heads, page_size, head_dim)
    if tuple(v_pages.shape) != expected:
        raise KernelShapeError(
            f"v_pages has shape {tuple(v_pages.shape)}, expected {expected} (v_transposed={v_transposed})"
        )


MFMA_HEAD_DIMS = (32, 64, 96, 128, 192, 256)
# what the plain attention kernel (and so the engine as a whole) takes: any even head size up
# to 256 (a rotation pairs dims, so an odd one has no meaning here)
ATTENTION_HEAD_DIM_STEP = 2
ATTENTION_MAX_HEAD_DIM = 256


def mfma_attention_supported(dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
    """Whether the matrix-core attention kernel takes this cache shape (else the plain kernel runs).

    Caches it takes store their values transposed inside each page.
    """
    return dtype == torch.bfloat16 and head_dim in MFMA_HEAD_DIMS and page_size % 16 == 0


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    """The current HIP stream's handle.  (Asked of torch's C layer directly where it offers
    that: the public `torch.cuda.current_stream()` builds a Python object per call, some 8 us,
    a fifth of the host's time in a step that is launched kernel by kernel.)"""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


# ----------------------------------------------------------------------------


def embed_gather(table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """`float32(table[ids]) * scale`: the start of the residual stream, [T, H] float32."""
    _need_cuda(table, ids)
    _need_contiguous("table", table)
    _need_contiguous("ids", ids)
    _need_int32("ids", ids)
    vocab, hidden = table.shape
    out = torch.empty((ids.numel(), hidden), dtype=torch.float32, device=table.device)
    lib = library.load()
    library.check(
        lib.mi_embed_gather(
            _dtype_code(table), _ptr(table), _ptr(ids), _ptr(out), ids.numel(), hidden, vocab,
            float(scale), _stream(),
        )
    )
    return out


def take_device_tokens(ids: torch.Tensor, from_rows: torch.Tensor, source: torch.Tensor, vocab: int) -> None:
    """In place: `ids[i] = source[from_rows[i]]` where `from_rows[i] >= 0` (all int32, on the device)."""
    _need_cuda(ids, from_rows, source)
    for name, t in (("ids", ids), ("from_rows", from_rows), ("source", source)):
        _need_contiguous(name, t)
        _need_int32(name, t)
    if ids.dim() != 1 or from_rows.shape != ids.shape or source.dim() != 1 or source.numel() == 0:
        raise KernelShapeError("take_device_tokens: ids and from_rows are [n], source is [rows >= 1]")
    lib = library.load()
    library.check(
        lib.mi_take_device_tokens(_ptr(ids), _ptr(from_rows), _ptr(source), ids.numel(), source.numel(), int(vocab), _stream())
    )


SLOT_WORDS = 8  # int32 words of a request's row in the table of state slots


def begin_step(
    ids: torch.Tensor,
    from_rows: torch.Tensor | None,
    source: torch.Tensor | None,
    vocab: int,
    slot_table: torch.Tensor | None,
    state_slots: torch.Tensor | None,
    seq_lens: torch.Tensor | None,
) -> None:
    """The first kernel of a step.  With `from_rows`: `take_device_tokens`.  With
    `slot_table` [slots, 8] int32: word 0 of row `state_slots[b]` becomes `seq_lens[b]`,
    the request's length after this step (negative slots are skipped)."""
    _need_cuda(ids, from_rows, source, slot_table, state_slots, seq_lens)
    for name, t in (("ids", ids), ("from_rows", from_rows), ("source", source), ("slot_table", slot_table),
                    ("state_slots", state_slots), ("seq_lens", seq_lens)):
        _need_contiguous(name, t)
        _need_int32(name, t)
    if from_rows is not None and (source is None or source.numel() == 0 or from_rows.shape != ids.shape):
        raise KernelShapeError("begin_step: from_rows is [n] like ids and needs a source of at least one row")
    num_requests = num_slots = 0
    if slot_table is not None:
        if slot_table.dim() != 2 or slot_table.shape[1] != SLOT_WORDS or state_slots is None or seq_lens is None:
            raise KernelShapeError(f"begin_step: the slot table is [slots, {SLOT_WORDS}] and needs state_slots and seq_lens")
        if state_slots.numel() != seq_lens.numel():
            raise KernelShapeError("begin_step: one slot id per request length")
        num_requests, num_slots = state_slots.numel(), slot_table.shape[0]
    lib = library.load()
    library.check(
        lib.mi_begin_step(
            _ptr(ids), _ptr(from_rows), _ptr(source), ids.numel(), 0 if source is None else source.numel(), int(vocab),
            _ptr(slot_table), _ptr(state_slots), _ptr(seq_lens), num_requests, num_slots, _stream(),
        )
    )


@dataclasses.dataclass
class PartialSums:
    """A product that has not been added up yet: `pieces` [S, T, N] float32 holds its sums
    over S ranges of K (`linear(..., partial_ok=True)`).  Their sum in order, rounded to
    `dtype`, is what `linear` returns otherwise; `add_rmsnorm` takes the pieces as they are
    and adds them on its way, anything else calls `finish()`."""

    pieces: torch.Tensor
    dtype: torch.dtype

    def finish(self) -> torch.Tensor:
        total = self.pieces[0]
        for piece in self.pieces[1:]:
            total = total + piece
        return total.to(self.dtype)


def add_rmsnorm(
    delta: torch.Tensor | PartialSums | None,
    residual: torch.Tensor,
    weight: torch.Tensor,
    eps: float,
    rows: torch.Tensor | None = None,
) -> torch.Tensor:
    """`residual += delta` in float32 (kept unless `rows`), then RMSNorm times `weight`.

    Returns [T, H] (or [len(rows), H]) in the dtype of `weight`.
    """
    pieces = None
    if isinstance(delta, PartialSums):
        if delta.dtype != weight.dtype:
            raise KernelShapeError(f"partial sums for {delta.dtype} meet a norm weight of {weight.dtype}")
        pieces, delta = delta.pieces, None
        _need_cuda(pieces)
        _need_contiguous("partial sums", pieces)
        if pieces.dtype != torch.float32 or pieces.dim() != 3 or tuple(pieces.shape[1:]) != tuple(residual.shape):
            raise KernelShapeError(
                f"partial sums {tuple(pieces.shape)} {pieces.dtype} do not fit residual {tuple(residual.shape)}"
            )
        if not 1 <= pieces.shape[0] <= 16:
            raise KernelShapeError(f"1 to 16 partial sums are taken, got {pieces.shape[0]}")
    _need_cuda(delta, residual, weight, rows)
    _need_contiguous("residual", residual)
    _need_contiguous("delta", delta)
    _need_contiguous("weight", weight)
    _need_contiguous("rows", rows)
    _need_int32("rows", rows)
    if residual.dtype != torch.float32:
        raise KernelShapeError(f"the residual stream is float32, got {residual.dtype}")
    tokens, hidden = residual.shape
    if weight.shape != (hidden,):
        raise KernelShapeError(f"norm weight has shape {tuple(weight.shape)}, expected ({hidden},)")
    if delta is not None and (delta.shape != residual.shape or delta.dtype != weight.dtype):
        raise KernelShapeError(
            f"delta {tuple(delta.shape)} {delta.dtype} does not fit residual "
            f"{tuple(residual.shape)} and weight dtype {weight.dtype}"
        )
    n_out = tokens if rows is None else rows.numel()
    out = torch.empty((n_out, hidden), dtype=weight.dtype, device=residual.device)
    lib = library.load()
    library.check(
        lib.mi_add_rmsnorm(
            _dtype_code(weight), _ptr(delta), _ptr(residual), _ptr(weight), _ptr(out), _ptr(rows),
            n_out, hidden, float(eps), _ptr(pieces), 0 if pieces is None else pieces.shape[0],
            tokens * hidden, _stream(),
        )
    )
    return out


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """`cos, sin` of `position * inv_freq`, both [T, len(inv_freq)] float32."""
    _need_cuda(positions, inv_freq)
    _need_contiguous("positions", positions)
    _need_contiguous("inv_freq", inv_freq)
    _need_int32("positions", positions)
    if inv_freq.dtype != torch.float32:
        raise KernelShapeError(f"inv_freq stays float32, got {inv_freq.dtype}")
    tokens, half = positions.numel(), inv_freq.numel()
    cos = torch.empty((tokens, half), dtype=torch.float32, device=positions.device)
    sin = torch.empty_like(cos)
    lib = library.load()
    library.check(
        lib.mi_rope_table(_ptr(positions), _ptr(inv_freq), _ptr(cos), _ptr(sin), tokens, half, _stream())
    )
    return cos, sin


def rope_kv_write(
    qkv: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    slot_mapping: torch.Tensor | None,
    k_pages: torch.Tensor | None,
    v_pages: torch.Tensor | None,
    *,
    q_heads: int,
    kv_heads: int,
    head_dim: int,
    rotary_dim: int,
    interleaved: bool = False,
    v_transposed: bool = False,
    v_head_dim: int | None = None,
) -> None:
    """Rotate q in place inside `qkv`; rotate k and write k, v into their page slots.
    `v_head_dim`: the width of a value head where it is not the keys' (`head_dim`).

    `qkv` is [T, (q_heads + 2*kv_heads) * head_dim] (rows may be strided); pages are
    [num_pages, kv_heads, page_size, head_dim], value pages
    [num_pages, kv_heads, head_dim, page_size] with `v_transposed`.  `kv_heads=0`
    rotates q only.
    """
    _need_cuda(qkv, cos, sin, slot_mapping, k_pages, v_pages)
    _need_contiguous("cos", cos)
    _need_contiguous("sin", sin)
    _need_contiguous("slot_mapping", slot_mapping)
    _need_contiguous("k_pages", k_pages)
    _need_contiguous("v_pages", v_pages)
    _need_int32("slot_mapping", slot_mapping)
    if qkv.dim() != 2 or qkv.stride(1) != 1:
        raise KernelShapeError(f"qkv must be [T, width] with unit inner stride, got {qkv.stride()}")
    tokens = qkv.shape[0]
    v_dim = head_dim if v_head_dim is None else int(v_head_dim)
    if qkv.shape[1] < (q_heads + kv_heads) * head_dim + kv_heads * v_dim:
        raise KernelShapeError(
            f"qkv rows hold {qkv.shape[1]} values, fewer than the q, k and v heads need: "
            f"{(q_heads + kv_heads) * head_dim + kv_heads * v_dim}"
        )
    if cos.shape != (tokens, rotary_dim // 2) or sin.shape != cos.shape or cos.dtype != torch.float32:
        raise KernelShapeError(
            f"cos/sin must be float32 [{tokens}, {rotary_dim // 2}], got {tuple(cos.shape)} {cos.dtype}"
        )
    page_size = num_pages = 0
    if kv_heads > 0 and slot_mapping is not None:
        if k_pages is None or v_pages is None:
            raise KernelShapeError("writing keys and values needs k_pages and v_pages")
        if k_pages.dtype != qkv.dtype or v_pages.dtype != qkv.dtype:
            raise KernelShapeError(f"pages are {k_pages.dtype}, activations {qkv.dtype}")
        if k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != head_dim:
            raise KernelShapeError(
                f"pages must be [num_pages, {kv_heads}, page_size, {head_dim}], got {tuple(k_pages.shape)}"
            )
        _check_v_pages(k_pages, v_pages, v_transposed, v_dim)
        if slot_mapping.numel() != tokens:
            raise KernelShapeError(f"slot_mapping has {slot_mapping.numel()} entries for {tokens} tokens")
        num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
    lib = library.load()
    library.check(
        lib.mi_rope_kv_write(
            _dtype_code(qkv), _ptr(qkv), qkv.stride(0), _ptr(cos), _ptr(sin), _ptr(slot_mapping),
            _ptr(k_pages), _ptr(v_pages), tokens, q_heads, kv_heads, head_dim, rotary_dim,
            int(interleaved), page_size, num_pages, int(v_transposed), v_dim, _stream(),
        )
    )


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """`silu(gate) * up` for rows laid out [gate | up]; returns [T, I]."""
    _need_cuda(gate_up)
    _need_contiguous("gate_up", gate_up)
    tokens, width = gate_up.shape
    if width % 2 != 0:
        raise KernelShapeError(f"gate_up rows must hold gate and up halves, got width {width}")
    out = torch.empty((tokens, width // 2), dtype=gate_up.dtype, device=gate_up.device)
    lib = library.load()
    library.check(
        lib.mi_silu_mul(_dtype_code(gate_up), _ptr(gate_up), _ptr(out), tokens, width // 2, _stream())
    )
    return out


def gemm_f32(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """`a @ w.T` in true float32: a [M, K], w [N, K] -> [M, N]."""
    _need_cuda(a, w)
    if a.dtype != torch.float32 or w.dtype != torch.float32:
        raise KernelShapeError(f"gemm_f32 takes float32, got {a.dtype} and {w.dtype}")
    if a.dim() != 2 or w.dim() != 2 or a.shape[1] != w.shape[1]:
        raise KernelShapeError(f"gemm_f32: shapes {tuple(a.shape)} and {tuple(w.shape)} do not fit")
    if a.stride(1) != 1 or w.stride(1) != 1:
        raise KernelShapeError("gemm_f32: rows must have unit inner stride")
    m, k = a.shape
    n = w.shape[0]
    c = torch.empty((m, n), dtype=torch.float32, device=a.device)
    lib = library.load()
    library.check(
        lib.mi_gemm_f32(_ptr(a), a.stride(0), _ptr(w), w.stride(0), _ptr(c), c.stride(0), m, n, k, _stream())
    )
    return c


SKINNY_MAX_ROWS = 16


def gemm_skinny_bf16(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """`a @ w.T` for at most 16 rows of bfloat16: a [M, K], w [N, K] -> [M, N], K % 32 == 0."""
    _need_cuda(a, w)
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelShapeError(f"gemm_skinny_bf16 takes bfloat16, got {a.dtype} and {w.dtype}")
    if a.dim() != 2 or w.dim() != 2 or a.shape[1] != w.shape[1]:
        raise KernelShapeError(f"gemm_skinny_bf16: shapes {tuple(a.shape)} and {tuple(w.shape)} do not fit")
    if a.stride(1) != 1 or w.stride(1) != 1:
        raise KernelShapeError("gemm_skinny_bf16: rows must have unit inner stride")
    m, k = a.shape
    n = w.shape[0]
    c = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    lib = library.load()
    library.check(
        lib.mi_gemm_skinny_bf16(_ptr(a), a.stride(0), _ptr(w), w.stride(0), _ptr(c), c.stride(0), m, n, k, _stream())
    )
    return c


def linear_f32_out(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """`x @ weight.T` as float32, whatever the operands' dtype: what an output head returns.

    Few bfloat16 rows: the weight-streaming kernel writes float32 itself (no cast launch); its
    values are those of `linear(...).float()`, rounded to bfloat16 on the way, so that a row's
    logits do not depend on how many rows its step had.  More rows: the vendor library's
    product, cast.  float32 operands: `gemm_f32`."""
    if x.dtype == torch.float32:
        return gemm_f32(x, weight)
    _need_cuda(x, weight)
    if (
        x.dtype == torch.bfloat16
        and weight.dtype == torch.bfloat16
        and x.dim() == 2
        and weight.dim() == 2
        and x.shape[1] == weight.shape[1]
        and x.stride(1) == 1
        and weight.stride(1) == 1
        and skinny_gemm_takes(x.shape[0], x.shape[1], x.stride(0), weight.stride(0))
    ):
        m, k = x.shape
        n = weight.shape[0]
        out = torch.empty((m, n), dtype=torch.float32, device=x.device)
        library.check(
            library.load().mi_gemm_skinny_f32out_bf16(
                _ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(out), out.stride(0), m, n, k, _stream()
            )
        )
        return out
    return torch.matmul(x, weight.t()).float()


def skinny_gemm_takes(m: int, k: int, lda: int, ldw: int, max_rows: int = SKINNY_MAX_ROWS) -> bool:
    return 1 <= m <= max_rows and k >= 32 and k % 32 == 0 and lda % 8 == 0 and ldw % 8 == 0


# The gated product and the q|k|v product with rotation and cache write take two tiles of 16
# rows: up to 32 rows they measured faster than the vendor product followed by `silu_mul` /
# `rope_kv_write` (8B sizes 12-21 %, 3B sizes 3-22 %), with 48 and 64 rows level or slower.
SKINNY_WIDE_MAX_ROWS = 32


PARTIAL_SUMS_MAX_ROWS = 128


def partial_sums_pay(m: int, n: int, k: int) -> bool:
    """Whether a product of these sizes is left as sums over ranges of K when its caller
    takes them (`linear(..., partial_ok=True)`).  Measured on MI355X, the product alone with
    weights from memory, microseconds whole / in pieces (whole = `gemm_skinny_bf16` up to
    16 rows, the vendor library above):

                                  8 rows    12 rows   16 rows   32 rows   64 rows
        4096 x 14336 (8B down)    22 / 23   26 / 24   28 / 24   34 / 25   39 / 28
        8192 x 28672 (70B down)   77 / 85   81 / 86   89 / 87  101 / 89  144 / 100
        3072 x 8192  (3B down)    12 / 18   14 / 18   16 / 19   17 / 20   23 / 22
        4096 x 4096  (8B o)        8 / 10    9 / 10   10 / 10   13 / 11   15 / 13
        3072 x 3072  (3B o)        7 / 8     7 / 8     8 / 8    11 / 9    16 / 11
        8192 x 8192  (70B o)      24 / 36   23 / 36   25 / 35   31 / 38   34 / 40

    and at 96 / 128 rows 63 / 75 against 36 / 39 (8B down), 22 / 24 against 16 / 18 (8B o),
    121 / 201 against 130 / 131 (70B down)

    (the norm that adds the pieces up costs about a microsecond more than one that does not),
    so: a long K from 11 rows on (15 with more than 4096 features), a small square-ish product
    where the weight-streaming kernel ends (17 rows), nothing else.  Whole decode steps at 8B
    sizes and 8 rows run 2.4 % faster with the down product whole, at 16 rows 2.6 % slower."""
    if not 5 <= m <= PARTIAL_SUMS_MAX_ROWS or n > 8192:
        return False
    if k >= 12288:
        return m >= (11 if n <= 4096 else 15)
    return m > SKINNY_MAX_ROWS and n <= 4096 and 2048 <= k <= 4096


def linear_partial_sums(x: torch.Tensor, weight: torch.Tensor) -> PartialSums:
    """`x @ weight.T` for up to 128 bfloat16 rows as float32 sums over ranges of K."""
    _need_cuda(x, weight)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or x.dim() != 2 or weight.dim() != 2:
        raise KernelShapeError("linear_partial_sums takes 2-D bfloat16 tensors")
    m, k = x.shape
    n = weight.shape[0]
    lib = library.load()
    if (
        weight.shape[1] != k
        or x.stride(1) != 1
        or weight.stride(1) != 1
        or not lib.mi_gemm_mid_bf16_supported(m, n, k, x.stride(0), weight.stride(0))
    ):
        raise KernelShapeError(
            f"linear_partial_sums takes 1 to 128 rows, K a multiple of 32, rows aligned to 16 bytes; "
            f"got x {tuple(x.shape)} strides {x.stride()}, weight {tuple(weight.shape)} strides {weight.stride()}"
        )
    ranges = lib.mi_gemm_mid_bf16_ranges(n, k)
    if ranges < 1:
        raise KernelShapeError("linear_partial_sums: cannot read the device's compute unit count")
    pieces = torch.empty((ranges, m, n), dtype=torch.float32, device=x.device)
    library.check(
        lib.mi_gemm_mid_partial_bf16(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(pieces), m, n, k, _stream())
    )
    return PartialSums(pieces, torch.bfloat16)


def linear(x: torch.Tensor, weight: torch.Tensor, partial_ok: bool = False) -> torch.Tensor | PartialSums:
    """`x @ weight.T` without bias.

    float32 runs the hand-written true-float32 kernel.  bfloat16 with at most 16
    rows (decode) runs the hand-written weight-streaming kernel; more rows go to
    the vendor GEMM library through torch, as the reference's engine does
    (distributed/linear.py:167, `F.linear` -> the vendor BLAS).
    With `partial_ok` the result may come as `PartialSums` where that pays
    (`partial_sums_pay`: up to 128 rows, few features, a long K).
    """
    if x.dtype == torch.float32:
        return gemm_f32(x, weight)
    _need_cuda(x, weight)
    plain = x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.dim() == 2 and weight.dim() == 2
    plain = plain and x.stride(1) == 1 and weight.stride(1) == 1 and weight.shape[1] == x.shape[1]
    if (
        partial_ok
        and plain
        and partial_sums_pay(x.shape[0], weight.shape[0], x.shape[1])
        and x.shape[1] % 32 == 0
        and x.stride(0) % 8 == 0
        and weight.stride(0) % 8 == 0
    ):
        return linear_partial_sums(x, weight)
    if (
        x.dtype == torch.bfloat16
        and x.dim() == 2
        and x.stride(1) == 1
        and weight.stride(1) == 1
        and skinny_gemm_takes(x.shape[0], x.shape[1], x.stride(0), weight.stride(0))
    ):
        return gemm_skinny_bf16(x, weight)
    return torch.matmul(x, weight.t())


def _scaled_rows_fit(x: "ScaledRows") -> bool:
    """Whether a product's kernel can apply the rows' factors of `x` itself."""
    return (
        x.values.dtype == torch.bfloat16
        and x.values.dim() == 2
        and x.values.shape[0] <= PENDING_PRODUCT_MAX_ROWS
        and x.sumsq.is_contiguous()
        and x.sumsq.shape[0] <= SCALED_ROWS_MAX_PIECES
    )


def scaled_rows_product_takes(rows: int, weight: torch.Tensor | None, norm_width: int) -> bool:
    """Whether a weight-streaming product with `weight` can take `rows` rows as `ScaledRows` of a
    norm over `norm_width` features: what a part answers its norm with before a step
    (`wants_scaled_rows`), so that no row is handed over in a form nobody has a kernel for."""
    if weight is None or weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.stride(1) != 1:
        return False
    if weight.shape[1] != norm_width or not skinny_gemm_takes(rows, norm_width, norm_width, weight.stride(0), PENDING_PRODUCT_MAX_ROWS):
        return False
    pieces = library.load().mi_gemm_skinny_addnorm_pieces(norm_width)
    return 0 < pieces <= SCALED_ROWS_MAX_PIECES


def qkv_rope_write_takes(
    x: "torch.Tensor | ScaledRows", weight: torch.Tensor, head_dim: int, rotary_dim: int, interleaved: bool
) -> bool:
    """Whether `qkv_rope_write` runs these operands: at most 32 bfloat16 rows (16 as
    `ScaledRows`), rotation of whole heads in half pairing, head size a multiple of 32."""
    max_rows = SKINNY_WIDE_MAX_ROWS
    if isinstance(x, ScaledRows):
        if not _scaled_rows_fit(x):
            return False
        x, max_rows = x.values, SKINNY_MAX_ROWS
    return (
        x.dtype == torch.bfloat16
        and weight.dtype == torch.bfloat16
        and x.dim() == 2
        and x.stride(1) == 1
        and weight.stride(1) == 1
        and skinny_gemm_takes(x.shape[0], x.shape[1], x.stride(0), weight.stride(0), max_rows)
        and not interleaved
        and rotary_dim == head_dim
        and head_dim % 32 == 0
    )


def qkv_rope_write(
    x: "torch.Tensor | ScaledRows",
    weight: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    slot_mapping: torch.Tensor | None,
    k_pages: torch.Tensor | None,
    v_pages: torch.Tensor | None,
    *,
    q_heads: int,
    kv_heads: int,
    head_dim: int,
    v_transposed: bool = False,
) -> torch.Tensor:
    """The stacked q|k|v projection, the rotary encoding and the cache write as ONE kernel.

    x [M <= 32, K] bfloat16, weight [(q_heads + 2*kv_heads)*head_dim, K]; returns the rotated
    queries [M, q_heads*head_dim]; rotated keys and values go to their slots.  `kv_heads=0`
    with the query rows of the weight alone projects and rotates queries only.  The result
    is that of `linear` followed by `rope_kv_write` (both round the product to bfloat16
    before rotating).  `x` may be `ScaledRows`: the rows' factors are then applied to the
    products' sums before they are rounded.
    """
    scaled = x if isinstance(x, ScaledRows) else None
    if scaled is not None:
        x = scaled.values
        _need_cuda(scaled.sumsq)
    _need_cuda(x, weight, cos, sin, slot_mapping, k_pages, v_pages)
    for name, t in (("cos", cos), ("sin", sin), ("slot_mapping", slot_mapping), ("k_pages", k_pages), ("v_pages", v_pages)):
        _need_contiguous(name, t)
    _need_int32("slot_mapping", slot_mapping)
    if not qkv_rope_write_takes(scaled if scaled is not None else x, weight, head_dim, head_dim, False):
        raise KernelShapeError(
            f"qkv_rope_write takes at most 32 bfloat16 rows and head sizes in steps of 32; got "
            f"x {tuple(x.shape)} {x.dtype}, head_dim={head_dim}"
        )
    m, k = x.shape
    if weight.shape != ((q_heads + 2 * kv_heads) * head_dim, k):
        raise KernelShapeError(f"qkv_rope_write: weight {tuple(weight.shape)} does not fit (q+2kv)*head_dim x {k}")
    if cos.shape != (m, head_dim // 2) or sin.shape != cos.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32:
        raise KernelShapeError(f"cos/sin must be float32 [{m}, {head_dim // 2}], got {tuple(cos.shape)} {cos.dtype}")
    page_size = num_pages = 0
    if kv_heads > 0:
        if slot_mapping is None or k_pages is None or v_pages is None:
            raise KernelShapeError("writing keys and values needs slot_mapping, k_pages and v_pages")
        if k_pages.dtype != torch.bfloat16 or v_pages.dtype != torch.bfloat16:
            raise KernelShapeError("qkv_rope_write writes bfloat16 pages")
        if k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != head_dim:
            raise KernelShapeError(
                f"k_pages must be [num_pages, {kv_heads}, page_size, {head_dim}], got {tuple(k_pages.shape)}"
            )
        _check_v_pages(k_pages, v_pages, v_transposed)
        if slot_mapping.numel() != m:
            raise KernelShapeError("slot_mapping needs one entry per row")
        num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
    q_out = torch.empty((m, q_heads * head_dim), dtype=torch.bfloat16, device=x.device)
    lib = library.load()
    rest = (
        _ptr(weight), weight.stride(0), _ptr(q_out), q_out.stride(0), _ptr(cos), _ptr(sin),
        _ptr(slot_mapping) if kv_heads > 0 else None, _ptr(k_pages) if kv_heads > 0 else None,
        _ptr(v_pages) if kv_heads > 0 else None, m, k, q_heads, kv_heads, head_dim, page_size, num_pages,
        int(v_transposed), _stream(),
    )
    if scaled is not None:
        library.check(
            lib.mi_gemm_skinny_rope_scaled_bf16(_ptr(x), x.stride(0), _ptr(scaled.sumsq), scaled.sumsq.shape[0], scaled.eps, *rest)
        )
    else:
        library.check(lib.mi_gemm_skinny_rope_bf16(_ptr(x), x.stride(0), *rest))
    return q_out


def linear_swiglu(x: "torch.Tensor | ScaledRows", gate_up_weight: torch.Tensor) -> torch.Tensor:
    """`silu(x @ gate.T) * (x @ up.T)` with `gate_up_weight` = [gate; up] stacked, [2I, K].

    bfloat16 with at most 32 rows runs as ONE hand-written kernel (the product with the
    activation in its last step); otherwise the product and `silu_mul` run in turn.
    Both ways round the two products to the element type before the activation, so given
    the same rows a token's result does not depend on which one ran.  `x` may be
    `ScaledRows`: the rows' factors are then applied to the sums of the two products (the same
    kernel with one more step), or to `x` first where that kernel does not take the shapes.
    Rows that come as `ScaledRows` were rounded before their factor was applied
    (`bf16(x * w)`, the factor then meets float32 sums), rows from a norm's own launch after
    it (`bf16(x * r * w)`): which way a step went shows in the last bit of a bfloat16 value.
    """
    rows, width = gate_up_weight.shape
    if rows % 2:
        raise KernelShapeError(f"linear_swiglu: stacked weight has an odd number of rows ({rows})")
    scaled = None
    if isinstance(x, ScaledRows):
        values = x.values
        if (
            _scaled_rows_fit(x)
            and gate_up_weight.dtype == torch.bfloat16
            and values.shape[1] == width
            and values.stride(1) == 1
            and gate_up_weight.stride(1) == 1
            and skinny_gemm_takes(values.shape[0], width, values.stride(0), gate_up_weight.stride(0))
        ):
            scaled, x = x, values
        else:
            x = x.finish()
    if (
        x.dtype == torch.bfloat16
        and gate_up_weight.dtype == torch.bfloat16
        and x.dim() == 2
        and x.shape[1] == width
        and x.stride(1) == 1
        and gate_up_weight.stride(1) == 1
        and skinny_gemm_takes(x.shape[0], x.shape[1], x.stride(0), gate_up_weight.stride(0), SKINNY_WIDE_MAX_ROWS)
    ):
        _need_cuda(x, gate_up_weight)
        m, n = x.shape[0], rows // 2
        out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
        lib = library.load()
        if scaled is not None:
            _need_cuda(scaled.sumsq)
            library.check(
                lib.mi_gemm_skinny_swiglu_scaled_bf16(
                    _ptr(x), x.stride(0), _ptr(scaled.sumsq), scaled.sumsq.shape[0], scaled.eps,
                    _ptr(gate_up_weight), gate_up_weight.stride(0), _ptr(out), out.stride(0), m, n, width, _stream(),
                )
            )
            return out
        library.check(
            lib.mi_gemm_skinny_swiglu_bf16(
                _ptr(x), x.stride(0), _ptr(gate_up_weight), gate_up_weight.stride(0), _ptr(out), out.stride(0),
                m, n, width, _stream(),
            )
        )
        return out
    return silu_mul(linear(x, gate_up_weight))


# Launch shapes of the matrix-core attention kernel: 128-row prefill blocks, two to a CU; decode
# blocks of 16 rows whose waves split the keys; and 256-row prefill blocks, one to a CU, which
# fetch every key and value tile half as often but need more blocks than there are CUs several
# times over, since the blocks of a causal prompt differ in length (one prompt, 8 key-value heads:
# 2,048 tokens 101 against 69 us, 8,192 tokens 670 against 716 us, 131,072 tokens 130 against 140 ms).
ATTN_SHAPE_PREFILL, ATTN_SHAPE_DECODE, ATTN_SHAPE_PREFILL_WIDE = 0, 1, 2
WIDE_PREFILL_MIN_BLOCKS = 512


def attention_splits(work_items: int, max_seq_len: int, target: int = 2048, min_keys: int = 256) -> int:
    """How many key ranges each work item is cut into so that the GPU is full.

    `work_items` blocks would run without splitting; `target` are wanted; a split
    keeps at least `min_keys` keys.
    """
    by_fill = max(1, target // max(1, work_items))
    by_len = max(1, max_seq_len // min_keys)
    return int(min(by_fill, by_len, 64))


@dataclasses.dataclass
class AttentionPieces:
    """An attention output that has not been combined yet: the results of `splits` key ranges
    per (token, head) as `attn_mfma` leaves them (`paged_attention(..., combine=False)`).
    `linear_from_attention` multiplies them with the output projection, combining on its way;
    `finish()` combines them as the attention would have."""

    part_acc: torch.Tensor  # [tokens * heads * splits, head_dim] float32
    part_ml: torch.Tensor  # [tokens * heads * splits, 2] float32: maximum (natural log units), sum
    splits: int
    tokens: int
    heads: int
    head_dim: int
    dtype: torch.dtype

    def finish(self) -> torch.Tensor:
        acc = self.part_acc.view(self.tokens, self.heads, self.splits, self.head_dim)
        ml = self.part_ml.view(self.tokens, self.heads, self.splits, 2)
        weight = torch.exp(ml[..., 0] - ml[..., 0].max(dim=-1, keepdim=True).values)
        total = (acc * weight[..., None]).sum(dim=2) / (ml[..., 1] * weight).sum(dim=-1, keepdim=True)
        return total.reshape(self.tokens, self.heads * self.head_dim).to(self.dtype)


def attention_pieces_pay(tokens: int, heads: int, head_dim: int) -> bool:
    """Whether a step of `tokens` single tokens leaves its attention uncombined for the output
    projection (`paged_attention(combine=False)` + `linear_from_attention`).  Every block of
    that projection reads all the key ranges' results (tokens x heads x ranges x head_dim
    floats), which costs more than the saved launch as soon as there are several tokens:
    measured at Llama-3.1-8B sizes, a single token runs 1 % faster this way, 8 tokens 6 %
    slower.  So: one token."""
    if tokens != 1 or heads < 1 or head_dim < 32 or head_dim % 32 != 0:
        return False
    return bool(library.load().mi_gemm_skinny_attn_bf16_supported(tokens, heads, head_dim))


def linear_from_attention(pieces: AttentionPieces, weight: torch.Tensor) -> torch.Tensor:
    """`attention output @ weight.T` for a few tokens, from the uncombined key ranges: one
    kernel instead of the combining kernel and the product."""
    _need_cuda(pieces.part_acc, pieces.part_ml, weight)
    k = pieces.heads * pieces.head_dim
    if (
        weight.dtype != torch.bfloat16
        or weight.dim() != 2
        or weight.shape[1] != k
        or weight.stride(1) != 1
        or weight.stride(0) % 8 != 0
        or not library.load().mi_gemm_skinny_attn_bf16_supported(pieces.tokens, pieces.heads, pieces.head_dim)
    ):
        raise KernelShapeError(
            f"linear_from_attention takes few tokens (tokens x heads*head_dim <= 32768), head_dim a multiple of 32 and a "
            f"bfloat16 weight [N, {k}]; got {pieces.tokens} tokens, head_dim {pieces.head_dim}, weight {tuple(weight.shape)} {weight.dtype}"
        )
    n = weight.shape[0]
    out = torch.empty((pieces.tokens, n), dtype=torch.bfloat16, device=weight.device)
    lib = library.load()
    library.check(
        lib.mi_gemm_skinny_attn_bf16(
            _ptr(pieces.part_acc), _ptr(pieces.part_ml), pieces.splits, pieces.heads, pieces.head_dim,
            _ptr(weight), weight.stride(0), _ptr(out), out.stride(0), pieces.tokens, n, _stream(),
        )
    )
    return out


PENDING_PRODUCT_MAX_ROWS = 16  # rows up to which a product is worth handing on unmade
SCALED_ROWS_MAX_PIECES = 256  # pieces of a row's sum of squares the consuming kernel adds up


def pending_product_pays(rows: int, n: int, k: int, partial_ok: bool) -> bool:
    """Whether a part hands its last product [rows, k] x [n, k] on unmade (`PendingProduct`)
    instead of making it: few rows, and not where the product is better left as sums over
    ranges of K (`partial_sums_pay`, if its caller takes those)."""
    return rows <= PENDING_PRODUCT_MAX_ROWS and not (partial_ok and partial_sums_pay(rows, n, k))


@dataclasses.dataclass
class PendingProduct:
    """`x @ weight.T` that has not been made yet: a part's contribution to the residual stream,
    handed to the norm that follows it so that one kernel can make the product, add it to the
    residual and begin the norm (`linear_add_norm`).  `x` is a matrix, or an attention output
    still lying in its key ranges.  Anything else calls `finish()`."""

    x: torch.Tensor | AttentionPieces
    weight: torch.Tensor

    def finish(self) -> torch.Tensor:
        if isinstance(self.x, AttentionPieces):
            return linear_from_attention(self.x, self.weight)
        return linear(self.x, self.weight)


@dataclasses.dataclass
class ScaledRows:
    """The output of an RMS norm but for each row's factor: `values` [T, H] = residual * norm
    weight (rounded to the element type), `sumsq` [pieces, T] float32 = sums of squares of
    the residual rows over `pieces` ranges of H.  Row t is still to be multiplied with
    rsqrt(sum(sumsq[:, t]) / H + eps); a product that consumes the rows does that to its own
    sums instead (`linear_swiglu`, `qkv_rope_write`), since the factor commutes with the product.  Anything
    else calls `finish()`."""

    values: torch.Tensor
    sumsq: torch.Tensor
    eps: float

    def finish(self) -> torch.Tensor:
        factor = torch.rsqrt(self.sumsq.sum(dim=0) / self.values.shape[1] + self.eps)
        return (self.values.float() * factor[:, None]).to(self.values.dtype)


def linear_add_norm_takes(pending: PendingProduct, residual: torch.Tensor, norm_weight: torch.Tensor) -> bool:
    """Whether `linear_add_norm` runs as one kernel: bfloat16, at most 16 rows, K a multiple
    of 32 (from key ranges: what `linear_from_attention` takes)."""
    weight = pending.weight
    if (
        weight.dtype != torch.bfloat16
        or norm_weight.dtype != torch.bfloat16
        or weight.dim() != 2
        or weight.stride(1) != 1
        or residual.dtype != torch.float32
        or not residual.is_cuda
        or not residual.is_contiguous()
        or tuple(norm_weight.shape) != (weight.shape[0],)
    ):
        return False
    x = pending.x
    rows = x.tokens if isinstance(x, AttentionPieces) else x.shape[0]
    if rows > PENDING_PRODUCT_MAX_ROWS:
        return False
    if isinstance(x, AttentionPieces):
        return (
            x.dtype == torch.bfloat16
            and x.heads * x.head_dim == weight.shape[1]
            and tuple(residual.shape) == (x.tokens, weight.shape[0])
            and weight.stride(0) % 8 == 0
            and bool(library.load().mi_gemm_skinny_attn_bf16_supported(x.tokens, x.heads, x.head_dim))
        )
    return (
        x.dtype == torch.bfloat16
        and x.dim() == 2
        and x.stride(1) == 1
        and x.shape[1] == weight.shape[1]
        and tuple(residual.shape) == (x.shape[0], weight.shape[0])
        and skinny_gemm_takes(x.shape[0], x.shape[1], x.stride(0), weight.stride(0))
    )


def linear_add_norm(pending: PendingProduct, residual: torch.Tensor, norm_weight: torch.Tensor, eps: float) -> ScaledRows:
    """`residual += x @ weight.T` (rounded to bfloat16 first, added in float32, kept) and the
    RMS norm of the sum but for the rows' factors, in one kernel (see `ScaledRows`)."""
    if not linear_add_norm_takes(pending, residual, norm_weight):
        raise KernelShapeError(
            "linear_add_norm takes bfloat16, at most 16 rows, K a multiple of 32, a float32 residual [rows, N] "
            f"and a norm weight [N]; got weight {tuple(pending.weight.shape)} {pending.weight.dtype}, "
            f"residual {tuple(residual.shape)} {residual.dtype}"
        )
    weight, x = pending.weight, pending.x
    _need_cuda(weight, residual, norm_weight)
    _need_contiguous("norm weight", norm_weight)
    rows, n = residual.shape
    k = weight.shape[1]
    lib = library.load()
    pieces = lib.mi_gemm_skinny_addnorm_pieces(n)
    if pieces <= 0:
        raise KernelShapeError(f"linear_add_norm: no block count for {n} features")
    values = torch.empty((rows, n), dtype=torch.bfloat16, device=residual.device)
    sumsq = torch.empty((pieces, rows), dtype=torch.float32, device=residual.device)
    if isinstance(x, AttentionPieces):
        _need_cuda(x.part_acc, x.part_ml)
        source = (None, 0, _ptr(x.part_acc), _ptr(x.part_ml), x.splits, x.heads, x.head_dim)
    else:
        _need_cuda(x)
        source = (_ptr(x), x.stride(0), None, None, 0, 0, 0)
    library.check(
        lib.mi_gemm_skinny_addnorm_bf16(
            *source, _ptr(weight), weight.stride(0), _ptr(residual), residual.stride(0), _ptr(norm_weight),
            _ptr(values), values.stride(0), _ptr(sumsq), rows, n, k, _stream(),
        )
    )
    return ScaledRows(values, sumsq, float(eps))


def paged_attention(
    q: torch.Tensor,
    k_pages: torch.Tensor,
    v_pages: torch.Tensor,
    block_table: torch.Tensor,
    token_request: torch.Tensor,
    positions: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    host_cu_seqlens_q: list[int] | None,
    *,
    q_heads: int,
    kv_heads: int,
    head_dim: int,
    scale: float,
    window: int | None,
    max_seq_len: int,
    v_transposed: bool = False,
    force_plain: bool = False,
    combine: bool = True,
    slopes: torch.Tensor | None = None,
    v_head_dim: int | None = None,
    sink_logit: float | None = None,
    chunk: int | None = None,
    sinks: torch.Tensor | None = None,
    softcap: float | None = None,
) -> torch.Tensor | AttentionPieces:
    """Causal attention of every token over its request's pages; returns [T, q_heads*head_dim].

    `v_head_dim`: value rows of another width than the keys' (the result is then
    [T, q_heads*v_head_dim]); with `v_pages=None` a value row is the first `v_head_dim` entries
    of its key row.  `sink_logit`: the softmax's denominator gets one more term
    exp(sink_logit), a sink that carries no value (both attention kernels know it; uncombined
    `AttentionPieces` do not).  Values of a width of their own run the plain kernel.

    `sinks` (float32 [q_heads], optional): a sink logit per query head instead of one for all
    (both kernels).  `softcap`: every scaled score becomes `softcap * tanh(score / softcap)` before
    slopes are applied (both kernels).

    `chunk`: a chunked mask: the token at position p sees only keys from `p // chunk * chunk` on
    (its own stretch of `chunk` positions, counted from the sequence's start); it combines with
    the causal order and with a window.  Uncombined `AttentionPieces` are not made with it.

    `slopes` (float32 [q_heads], optional): the score of head h for the key at position j
    seen from position p gets `slopes[h] * (j - p)` added before the softmax (both kernels).

    With `combine=False` a step of single tokens whose keys are cut into ranges (the
    matrix-core kernel) comes back as `AttentionPieces`, for `linear_from_attention`.

    `q` is [T, >= q_heads*head_dim] with the rotated queries in its first columns
    (rows may be strided, so the merged projection's buffer can be passed as it is).
    Tokens of a request are consecutive and sit at consecutive positions;
    `cu_seqlens_q` (device) and `host_cu_seqlens_q` give the request boundaries.
    `host_cu_seqlens_q=None`: the boundaries are known on the device only (a step that is
    recorded once and replayed with other boundaries); the launch is then shaped by the number
    of tokens and requests alone, with as many tiles as any division of the tokens among the
    requests can need, and requests without tokens are allowed.
    bfloat16 caches with transposed values run on the matrix cores; everything else
    (float32, other head or page sizes) runs the plain kernel.
    """
    if chunk is not None and chunk <= 0:
        raise KernelShapeError(f"a chunked mask needs a positive chunk, got {chunk}")
    if sinks is not None:
        _need_cuda(sinks)
        _need_contiguous("sinks", sinks)
        if sinks.dtype != torch.float32 or sinks.numel() != q_heads:
            raise KernelShapeError(f"sinks must be float32 [{q_heads}], got {sinks.dtype} x {sinks.numel()}")
        if sink_logit is not None:
            raise KernelShapeError("a sink logit for all heads or one per head, not both")
    has_sink = sink_logit is not None or sinks is not None
    if v_pages is None or (v_head_dim is not None and v_head_dim != head_dim) or (
        (has_sink or chunk is not None or softcap is not None) and not v_transposed
    ):
        return _paged_attention_general(
            q, k_pages, v_pages, block_table, token_request, positions, q_heads=q_heads, kv_heads=kv_heads,
            head_dim=head_dim, v_head_dim=head_dim if v_head_dim is None else int(v_head_dim), scale=scale,
            window=window, max_seq_len=max_seq_len, v_transposed=v_transposed, slopes=slopes, sink_logit=sink_logit,
            chunk=chunk, sinks=sinks, softcap=softcap,
        )
    _need_cuda(q, k_pages, v_pages, block_table, token_request, positions, cu_seqlens_q)
    for name, t in (("k_pages", k_pages), ("v_pages", v_pages), ("block_table", block_table),
                    ("token_request", token_request), ("positions", positions),
                    ("cu_seqlens_q", cu_seqlens_q)):
        _need_contiguous(name, t)
    for name, t in (("block_table", block_table), ("token_request", token_request),
                    ("positions", positions), ("cu_seqlens_q", cu_seqlens_q)):
        _need_int32(name, t)
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < q_heads * head_dim:
        raise KernelShapeError(f"q must be [T, >= {q_heads * head_dim}] with unit inner stride")
    if k_pages.dtype != q.dtype or v_pages.dtype != q.dtype:
        raise KernelShapeError(f"pages are {k_pages.dtype}, queries {q.dtype}")
    if k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != head_dim:
        raise KernelShapeError(
            f"pages must be [num_pages, {kv_heads}, page_size, {head_dim}], got {tuple(k_pages.shape)}"
        )
    _check_v_pages(k_pages, v_pages, v_transposed)
    tokens = q.shape[0]
    if token_request.numel() != tokens or positions.numel() != tokens:
        raise KernelShapeError("token_request and positions need one entry per token")
    if block_table.dim() != 2:
        raise KernelShapeError("block_table must be [requests, max_blocks]")
    num_requests = block_table.shape[0]
    if cu_seqlens_q.numel() != num_requests + 1 or (
        host_cu_seqlens_q is not None and len(host_cu_seqlens_q) != num_requests + 1
    ):
        raise KernelShapeError("cu_seqlens_q needs one more entry than there are requests")
    if host_cu_seqlens_q is not None and host_cu_seqlens_q[-1] != tokens:
        raise KernelShapeError(f"cu_seqlens_q ends at {host_cu_seqlens_q[-1]}, but there are {tokens} tokens")
    num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
    out = torch.empty((tokens, q_heads * head_dim), dtype=q.dtype, device=q.device)
    lib = library.load()
    group = q_heads // kv_heads

    use_mfma = v_transposed and not force_plain
    if v_transposed and not mfma_attention_supported(q.dtype, head_dim, page_size):
        raise KernelShapeError(
            f"transposed value pages need the matrix-core kernel, which does not take "
            f"{q.dtype}, head_dim={head_dim}, page_size={page_size}"
        )
    if v_transposed and force_plain:
        raise KernelShapeError("the plain attention kernel reads value pages that are not transposed")
    if slopes is not None:
        _need_cuda(slopes)
        _need_contiguous("slopes", slopes)
        if slopes.dtype != torch.float32 or slopes.numel() != q_heads:
            raise KernelShapeError(f"slopes must be float32 [{q_heads}], got {slopes.dtype} x {slopes.numel()}")

    def partials(splits: int, rows: int = tokens) -> tuple[torch.Tensor | None, torch.Tensor | None]:
        if splits == 1:
            return None, None
        return (
            torch.empty((rows * q_heads * splits, head_dim), dtype=torch.float32, device=q.device),
            torch.empty((rows * q_heads * splits, 2), dtype=torch.float32, device=q.device),
        )

    if use_mfma and host_cu_seqlens_q is None:
        # boundaries on the device only: one launch in the prefill shape, every wave finding its
        # tile's request itself; a request of q tokens has ceil(q / tile) tiles, at most
        # tokens // tile + requests of them in all, and the tiles past the real ones find nothing
        shape = ATTN_SHAPE_PREFILL
        tokens_per_tile = lib.mi_attn_mfma_tokens_per_tile(q_heads, kv_heads, shape)
        num_tiles = tokens // tokens_per_tile + num_requests
        head_blocks = -(-group // min(group, 128))
        splits = min(16, attention_splits(num_tiles * kv_heads * head_blocks, max_seq_len, target=512, min_keys=128))
        part_acc, part_ml = partials(splits)
        library.check(
            lib.mi_attn_mfma(
                _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(block_table), block_table.shape[1],
                _ptr(cu_seqlens_q), _ptr(positions), num_requests, tokens, num_tiles, _ptr(out), out.stride(0),
                _ptr(part_acc), _ptr(part_ml), q_heads, kv_heads, head_dim, page_size, num_pages, float(scale),
                int(window or 0), splits, shape, 0, 0, 1, int(has_sink), float(sink_logit or 0.0),
                int(chunk or 0), _ptr(sinks), _ptr(slopes), float(softcap or 0.0), _stream(),
            )
        )
        return out
    if use_mfma:
        q_lens = [host_cu_seqlens_q[b + 1] - host_cu_seqlens_q[b] for b in range(num_requests)]
        max_blocks = block_table.shape[1]

        def run(first: int, last: int, leave_pieces: bool = False) -> AttentionPieces | None:
            """Requests [first, last) of the step in one launch."""
            lens = q_lens[first:last]
            count = last - first
            first_token = host_cu_seqlens_q[first]
            run_tokens = host_cu_seqlens_q[last] - first_token
            decode_only = max(lens) <= 1
            shape = ATTN_SHAPE_DECODE if decode_only else ATTN_SHAPE_PREFILL
            if not decode_only and head_dim <= 128:
                wide_tile = lib.mi_attn_mfma_tokens_per_tile(q_heads, kv_heads, ATTN_SHAPE_PREFILL_WIDE)
                wide_blocks = sum(-(-n // wide_tile) for n in lens) * kv_heads * -(-group // min(group, 256))
                if wide_blocks >= WIDE_PREFILL_MIN_BLOCKS:
                    shape = ATTN_SHAPE_PREFILL_WIDE
            tokens_per_tile = lib.mi_attn_mfma_tokens_per_tile(q_heads, kv_heads, shape)
            # 2: exactly one token per request (the kernel then needs no request boundaries)
            one_tile_per_request = 2 if (decode_only and min(lens) == 1) else int(max(lens) <= tokens_per_tile)
            num_tiles = count if one_tile_per_request else sum(-(-n // tokens_per_tile) for n in lens)
            rows = {ATTN_SHAPE_DECODE: 16, ATTN_SHAPE_PREFILL: 128, ATTN_SHAPE_PREFILL_WIDE: 256}[shape]
            head_blocks = -(-group // min(group, rows))
            # decode blocks are register-heavy (about one per CU at a time measured best at
            # batch 1, 8 and 64) and a wide prefill block fills a CU; prefill blocks run two to a CU
            target = 512 if shape == ATTN_SHAPE_PREFILL else 256
            # few requests with long contexts are cut finer (measured at batch 1: 128k keys
            # run 19 % faster in 32 ranges than in 16, 3k keys 4 % slower)
            most = 16 if max_seq_len < 8192 else 32
            splits = min(most, attention_splits(num_tiles * kv_heads * head_blocks, max_seq_len, target=target, min_keys=128))
            part_acc, part_ml = partials(splits, first_token + run_tokens)
            library.check(
                lib.mi_attn_mfma(
                    _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages),
                    _ptr(block_table) + 4 * first * max_blocks, max_blocks,
                    _ptr(cu_seqlens_q) + 4 * first, _ptr(positions), count, run_tokens,
                    num_tiles, _ptr(out), out.stride(0), _ptr(part_acc), _ptr(part_ml), q_heads, kv_heads,
                    head_dim, page_size, num_pages, float(scale), int(window or 0), splits,
                    shape, int(one_tile_per_request), first_token,
                    0 if (leave_pieces and splits > 1) else 1, int(has_sink), float(sink_logit or 0.0),
                    int(chunk or 0), _ptr(sinks), _ptr(slopes), float(softcap or 0.0), _stream(),
                )
            )
            if leave_pieces and splits > 1:
                return AttentionPieces(part_acc, part_ml, splits, run_tokens, q_heads, head_dim, q.dtype)
            return None

        # Leading requests that bring a single token (a scheduler puts its decoding requests
        # first) run in the decode shape, where waves split the keys; inside the 128-row
        # prefill shape each of them would walk all its keys in one block, with 3 % of the
        # rows in use.
        leading_single = 0
        while leading_single < num_requests and q_lens[leading_single] == 1:
            leading_single += 1
        if 0 < leading_single < num_requests:
            run(0, leading_single)
            run(leading_single, num_requests)
        else:
            pieces = run(0, num_requests, leave_pieces=not combine and not has_sink and chunk is None
                         and leading_single == num_requests)
            if pieces is not None:
                return pieces
        return out

    assert chunk is None  # (a chunked mask on plain pages has gone to the general entry point above)
    splits = attention_splits(tokens * kv_heads * math.ceil(group / 4), max_seq_len)
    part_acc, part_ml = partials(splits)
    library.check(
        lib.mi_attn_generic(
            _dtype_code(q), _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
            block_table.shape[1], _ptr(token_request), _ptr(positions), _ptr(out), out.stride(0),
            _ptr(part_acc), _ptr(part_ml), tokens, q_heads, kv_heads, head_dim, page_size, num_pages,
            float(scale), int(window or 0), splits, _ptr(slopes), _stream(),
        )
    )
    return out


GENERAL_ATTENTION_MAX_KEY_DIM = 1024
GENERAL_ATTENTION_MAX_VALUE_DIM = 512


def _paged_attention_general(
    q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor | None, block_table: torch.Tensor,
    token_request: torch.Tensor, positions: torch.Tensor, *, q_heads: int, kv_heads: int, head_dim: int,
    v_head_dim: int, scale: float, window: int | None, max_seq_len: int, v_transposed: bool,
    slopes: torch.Tensor | None, sink_logit: float | None, chunk: int | None = None,
    sinks: torch.Tensor | None = None, softcap: float | None = None,
) -> torch.Tensor:
    """The plain attention kernel with everything it can be told: see `paged_attention`."""
    _need_cuda(q, k_pages, v_pages, block_table, token_request, positions, slopes, sinks)
    if softcap is not None and not softcap > 0:
        raise KernelShapeError(f"a cap on the scores must be positive, got {softcap}")
    for name, t in (("k_pages", k_pages), ("v_pages", v_pages), ("block_table", block_table),
                    ("token_request", token_request), ("positions", positions), ("slopes", slopes)):
        _need_contiguous(name, t)
    for name, t in (("block_table", block_table), ("token_request", token_request), ("positions", positions)):
        _need_int32(name, t)
    if v_transposed:
        raise KernelShapeError("the plain attention kernel reads value pages that are not transposed")
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < q_heads * head_dim:
        raise KernelShapeError(f"q must be [T, >= {q_heads * head_dim}] with unit inner stride")
    if k_pages.dtype != q.dtype or k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != head_dim:
        raise KernelShapeError(
            f"key pages must be {q.dtype} [num_pages, {kv_heads}, page_size, {head_dim}], got {k_pages.dtype} {tuple(k_pages.shape)}"
        )
    num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
    if v_pages is None:
        if not 0 < v_head_dim <= head_dim:
            raise KernelShapeError(f"a value row inside a key row of {head_dim} cannot be {v_head_dim} wide")
        values, v_row_stride = k_pages, head_dim
    else:
        if v_pages.dtype != q.dtype or tuple(v_pages.shape) != (num_pages, kv_heads, page_size, v_head_dim):
            raise KernelShapeError(
                f"value pages must be {q.dtype} {(num_pages, kv_heads, page_size, v_head_dim)}, got {v_pages.dtype} {tuple(v_pages.shape)}"
            )
        values, v_row_stride = v_pages, v_head_dim
    if head_dim % 2 or v_head_dim % 2 or head_dim > GENERAL_ATTENTION_MAX_KEY_DIM or v_head_dim > GENERAL_ATTENTION_MAX_VALUE_DIM:
        raise KernelShapeError(
            f"the plain attention kernel takes even key rows up to {GENERAL_ATTENTION_MAX_KEY_DIM} and even value rows "
            f"up to {GENERAL_ATTENTION_MAX_VALUE_DIM}, got {head_dim} and {v_head_dim}"
        )
    tokens = q.shape[0]
    if token_request.numel() != tokens or positions.numel() != tokens or block_table.dim() != 2:
        raise KernelShapeError("token_request and positions need one entry per token, block_table is [requests, max_blocks]")
    if slopes is not None and (slopes.dtype != torch.float32 or slopes.numel() != q_heads):
        raise KernelShapeError(f"slopes must be float32 [{q_heads}], got {slopes.dtype} x {slopes.numel()}")
    out = torch.empty((tokens, q_heads * v_head_dim), dtype=q.dtype, device=q.device)
    group = q_heads // kv_heads
    # (no row sees more keys than a chunk holds)
    splits = attention_splits(tokens * kv_heads * math.ceil(group / 4), min(max_seq_len, chunk) if chunk else max_seq_len)
    part_acc = part_ml = None
    if splits > 1:
        part_acc = torch.empty((tokens * q_heads * splits, v_head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((tokens * q_heads * splits, 2), dtype=torch.float32, device=q.device)
    library.check(
        library.load().mi_attn_general(
            _dtype_code(q), _ptr(q), q.stride(0), _ptr(k_pages), _ptr(values), _ptr(block_table), block_table.shape[1],
            _ptr(token_request), _ptr(positions), _ptr(out), out.stride(0), _ptr(part_acc), _ptr(part_ml), tokens,
            q_heads, kv_heads, head_dim, v_head_dim, v_row_stride, page_size, num_pages, float(scale), int(window or 0),
            splits, _ptr(slopes), int(sink_logit is not None or sinks is not None), float(sink_logit or 0.0), int(chunk or 0),
            float(softcap or 0.0), _ptr(sinks), _stream(),
        )
    )
    return out


# ----------------------------------------------------------------------------
# sublayers that add their own normed output to the stream, and what goes with them
# ----------------------------------------------------------------------------


def _need_f32(name: str, t: torch.Tensor | None) -> None:
    if t is not None and t.dtype != torch.float32:
        raise KernelShapeError(f"{name} stays float32, got {t.dtype}")


def embed_sinusoid(
    table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor, scale: float,
    want_cast: bool = False,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """`float32(table[ids]) * scale + wave(positions)`: column 2i of the wave is sin(p * freq[i]),
    column 2i+1 the cosine.  `freq` is float64 [ceil(H/2)].  Returns the float32 stream [T, H] and,
    with `want_cast`, the same rows in the table's dtype."""
    _need_cuda(table, ids, positions, freq)
    for name, t in (("table", table), ("ids", ids), ("positions", positions), ("freq", freq)):
        _need_contiguous(name, t)
    _need_int32("ids", ids)
    _need_int32("positions", positions)
    vocab, hidden = table.shape
    if freq.dtype != torch.float64 or freq.numel() != (hidden + 1) // 2:
        raise KernelShapeError(f"freq must be float64 [{(hidden + 1) // 2}], got {freq.dtype} x {freq.numel()}")
    if positions.numel() != ids.numel():
        raise KernelShapeError("embed_sinusoid: one position per token id")
    out = torch.empty((ids.numel(), hidden), dtype=torch.float32, device=table.device)
    cast = torch.empty((ids.numel(), hidden), dtype=table.dtype, device=table.device) if want_cast else None
    library.check(
        library.load().mi_embed_sinusoid(
            _dtype_code(table), _ptr(table), _ptr(ids), _ptr(positions), _ptr(freq), _ptr(out), _ptr(cast),
            ids.numel(), hidden, vocab, float(scale), _stream(),
        )
    )
    return out, cast


def norm_scale_add(
    y: torch.Tensor, residual: torch.Tensor, gain: torch.Tensor | None, scale: torch.Tensor | None, eps: float,
    want_cast: bool = False,
) -> torch.Tensor | None:
    """`residual += y * rsqrt(mean(y^2) + eps) * gain * scale` row by row, in place (float32).
    `gain`: one float32 number or None; `scale`: float32 [H] or None.  With `want_cast` the new
    rows are returned in the dtype of `y` as well."""
    _need_cuda(y, residual, gain, scale)
    _need_contiguous("residual", residual)
    _need_contiguous("scale", scale)
    _need_f32("residual", residual)
    _need_f32("gain", gain)
    _need_f32("scale", scale)
    if y.dim() != 2 or y.stride(1) != 1 or tuple(y.shape) != tuple(residual.shape):
        raise KernelShapeError(f"norm_scale_add: y {tuple(y.shape)} does not fit the stream {tuple(residual.shape)}")
    tokens, hidden = residual.shape
    if gain is not None and gain.numel() != 1:
        raise KernelShapeError(f"norm_scale_add: the gain is one number, got {gain.numel()}")
    if scale is not None and scale.numel() != hidden:
        raise KernelShapeError(f"norm_scale_add: the scale has {scale.numel()} entries for {hidden} columns")
    cast = torch.empty((tokens, hidden), dtype=y.dtype, device=y.device) if want_cast else None
    library.check(
        library.load().mi_norm_scale_add(
            _dtype_code(y), _ptr(y), y.stride(0), _ptr(residual), _ptr(gain), _ptr(scale), _ptr(cast), tokens, hidden,
            float(eps), _stream(),
        )
    )
    return cast


def cast_rows(residual: torch.Tensor) -> torch.Tensor:
    """The float32 stream rounded to bfloat16."""
    _need_cuda(residual)
    _need_contiguous("residual", residual)
    _need_f32("residual", residual)
    out = torch.empty(residual.shape, dtype=torch.bfloat16, device=residual.device)
    library.check(library.load().mi_cast_rows(_ptr(residual), _ptr(out), residual.numel(), _stream()))
    return out


GATED_SCAN_CHUNK = 32  # rows of a chunk of the chunked recurrence where the tiled kernels do not take the shapes
GATED_SCAN_SEQUENTIAL_ROWS = 128  # portions up to this many rows are walked by one thread a column


def gated_scan(
    zxg: torch.Tensor, bias_z: torch.Tensor, bias_x: torch.Tensor, state: torch.Tensor, cu_seqlens: torch.Tensor,
    slots: torch.Tensor, max_rows: int | None,
) -> torch.Tensor:
    """minGRU over the rows of a step.  `zxg` [T, 3W] holds the projections [z | x | g] of every
    token; request b owns rows `cu_seqlens[b]..cu_seqlens[b+1]` and the state row `state[slots[b]]`
    (float32 [slots + 1, W], rows may be strided; a negative slot means the last row, which is nobody's).  Returns
    `S_t * silu(g_t)` [T, W]; the state rows are advanced in place.  `max_rows`: the most rows a
    request brings, if the host knows (long portions then run chunk by chunk in parallel)."""
    _need_cuda(zxg, bias_z, bias_x, state, cu_seqlens, slots)
    for name, t in (("bias_z", bias_z), ("bias_x", bias_x), ("cu_seqlens", cu_seqlens), ("slots", slots)):
        _need_contiguous(name, t)
    _need_int32("cu_seqlens", cu_seqlens)
    _need_int32("slots", slots)
    for name, t in (("bias_z", bias_z), ("bias_x", bias_x), ("state", state)):
        _need_f32(name, t)
    if zxg.dim() != 2 or zxg.stride(1) != 1 or zxg.shape[1] % 3 != 0:
        raise KernelShapeError(f"gated_scan: rows hold [z | x | g], got {tuple(zxg.shape)} strides {zxg.stride()}")
    tokens, width = zxg.shape[0], zxg.shape[1] // 3
    requests = slots.numel()
    if cu_seqlens.numel() != requests + 1 or bias_z.numel() != width or bias_x.numel() != width:
        raise KernelShapeError("gated_scan: one more boundary than requests, one bias per column")
    if state.dim() != 2 or state.shape[1] != width or state.shape[0] < 2 or state.stride(1) != 1:
        raise KernelShapeError(f"gated_scan: state is [slots + 1, {width}] with unit inner stride, got {tuple(state.shape)}")
    out = torch.empty((tokens, width), dtype=zxg.dtype, device=zxg.device)
    chunk = chunks = 0
    summaries = None
    if max_rows is not None and max_rows > GATED_SCAN_SEQUENTIAL_ROWS:
        chunk = GATED_SCAN_CHUNK
        if width % 8 == 0 and zxg.stride(0) % 8 == 0:  # what the tiled kernels take: their chunk is theirs to say
            chunk = library.load().mi_gated_scan_tile_rows(_dtype_code(zxg))
        chunks = -(-max_rows // chunk)
        summaries = torch.empty((requests, chunks + 1, 2, width), dtype=torch.float32, device=zxg.device)
    library.check(
        library.load().mi_gated_scan(
            _dtype_code(zxg), _ptr(zxg), zxg.stride(0), _ptr(bias_z), _ptr(bias_x), _ptr(state), state.stride(0), _ptr(cu_seqlens),
            _ptr(slots), _ptr(out), out.stride(0), requests, width, state.shape[0] - 1, chunk, chunks, _ptr(summaries),
            _stream(),
        )
    )
    return out


def qk_norm_kv_write(
    qk: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor | None, slot_mapping: torch.Tensor | None,
    k_pages: torch.Tensor | None, v_pages: torch.Tensor | None, *, q_width: int, kv_heads: int, head_dim: int,
    eps: float, v_transposed: bool = False,
) -> None:
    """`qk` [T, q_width + kv_heads*head_dim]: q is normed in place over its whole width
    (`q * rsqrt(mean(q^2) + eps) * q_weight`); k, normed the same way with `k_weight`, goes to its
    key-page slot and k as it came to the value-page slot.  `kv_heads=0`: q only."""
    _need_cuda(qk, q_weight, k_weight, slot_mapping, k_pages, v_pages)
    for name, t in (("q_weight", q_weight), ("k_weight", k_weight), ("slot_mapping", slot_mapping),
                    ("k_pages", k_pages), ("v_pages", v_pages)):
        _need_contiguous(name, t)
    _need_int32("slot_mapping", slot_mapping)
    _need_f32("q_weight", q_weight)
    _need_f32("k_weight", k_weight)
    if qk.dim() != 2 or qk.stride(1) != 1 or qk.shape[1] < q_width + kv_heads * head_dim:
        raise KernelShapeError(f"qk_norm_kv_write: rows hold q and k, got {tuple(qk.shape)} strides {qk.stride()}")
    if q_weight.numel() != q_width or (kv_heads > 0 and (k_weight is None or k_weight.numel() != kv_heads * head_dim)):
        raise KernelShapeError("qk_norm_kv_write: one norm weight per column of q and of k")
    tokens = qk.shape[0]
    page_size = num_pages = 0
    if kv_heads > 0:
        if slot_mapping is None or k_pages is None or v_pages is None:
            raise KernelShapeError("writing keys and values needs slot_mapping, k_pages and v_pages")
        if k_pages.dtype != qk.dtype or v_pages.dtype != qk.dtype:
            raise KernelShapeError(f"pages are {k_pages.dtype}, activations {qk.dtype}")
        if k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != head_dim:
            raise KernelShapeError(f"pages must be [num_pages, {kv_heads}, page_size, {head_dim}], got {tuple(k_pages.shape)}")
        _check_v_pages(k_pages, v_pages, v_transposed)
        if slot_mapping.numel() != tokens:
            raise KernelShapeError(f"slot_mapping has {slot_mapping.numel()} entries for {tokens} tokens")
        num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
    library.check(
        library.load().mi_qk_norm_kv_write(
            _dtype_code(qk), _ptr(qk), qk.stride(0), _ptr(q_weight), _ptr(k_weight),
            _ptr(slot_mapping) if kv_heads > 0 else None, _ptr(k_pages) if kv_heads > 0 else None,
            _ptr(v_pages) if kv_heads > 0 else None, tokens, q_width, kv_heads, head_dim, page_size, num_pages,
            int(v_transposed), float(eps), _stream(),
        )
    )


def poly_norm(z: torch.Tensor, coefficients: torch.Tensor, eps: float) -> torch.Tensor:
    """`a N(z) + b N(z^2) + c N(z^3) + e` row by row, N(v) = v / sqrt(mean(v^2) + eps);
    `coefficients` = (a, b, c, e) float32."""
    _need_cuda(z, coefficients)
    _need_contiguous("coefficients", coefficients)
    _need_f32("coefficients", coefficients)
    if z.dim() != 2 or z.stride(1) != 1 or coefficients.numel() != 4:
        raise KernelShapeError(f"poly_norm: z is [T, width], four coefficients; got {tuple(z.shape)}, {coefficients.numel()}")
    out = torch.empty(z.shape, dtype=z.dtype, device=z.device)
    library.check(
        library.load().mi_poly_norm(
            _dtype_code(z), _ptr(z), z.stride(0), _ptr(coefficients), _ptr(out), out.stride(0), z.shape[0], z.shape[1],
            float(eps), _stream(),
        )
    )
    return out


def gated_table_rows(gate: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, first_col: int) -> torch.Tensor:
    """`gelu_tanh(gate) * table[ids, first_col : first_col + width]` for `gate` [T, width]."""
    _need_cuda(gate, table, ids)
    _need_contiguous("table", table)
    _need_contiguous("ids", ids)
    _need_int32("ids", ids)
    if gate.dim() != 2 or gate.stride(1) != 1 or table.dim() != 2 or table.dtype != gate.dtype:
        raise KernelShapeError("gated_table_rows: gate is [T, width], the table [vocab, columns] of the same dtype")
    tokens, width = gate.shape
    if ids.numel() != tokens or first_col < 0 or first_col + width > table.shape[1]:
        raise KernelShapeError(
            f"gated_table_rows: columns {first_col}..{first_col + width} of a table with {table.shape[1]}, {ids.numel()} ids for {tokens} rows"
        )
    out = torch.empty((tokens, width), dtype=gate.dtype, device=gate.device)
    library.check(
        library.load().mi_gated_table_rows(
            _dtype_code(gate), _ptr(gate), gate.stride(0), _ptr(table), table.stride(0), _ptr(ids), _ptr(out), tokens,
            width, int(first_col), table.shape[0], _stream(),
        )
    )
    return out


def linear_gru_takes(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether `linear_gru` runs these operands: at most 16 bfloat16 rows, K a multiple of 32."""
    return (
        x.dtype == torch.bfloat16
        and weight.dtype == torch.bfloat16
        and x.dim() == 2
        and weight.dim() == 2
        and weight.shape[0] % 3 == 0
        and x.shape[1] == weight.shape[1]
        and x.stride(1) == 1
        and weight.stride(1) == 1
        and skinny_gemm_takes(x.shape[0], x.shape[1], x.stride(0), weight.stride(0))
    )


def linear_gru(
    x: torch.Tensor, weight: torch.Tensor, bias_z: torch.Tensor, bias_x: torch.Tensor, state: torch.Tensor, slots: torch.Tensor
) -> torch.Tensor:
    """The stacked projection [z; x; g] of a minGRU and ONE step of its recurrence as one kernel,
    for a step in which every request brings exactly one token: row b of `x` belongs to the
    request whose state row is `state[slots[b]]`.  The values are those of `linear` followed by
    `gated_scan`, bit for bit (both round the products to bfloat16 first)."""
    if not linear_gru_takes(x, weight):
        raise KernelShapeError(f"linear_gru takes at most 16 bfloat16 rows and K in steps of 32; got x {tuple(x.shape)} {x.dtype}")
    _need_cuda(x, weight, bias_z, bias_x, state, slots)
    for name, t in (("bias_z", bias_z), ("bias_x", bias_x), ("slots", slots)):
        _need_contiguous(name, t)
    _need_int32("slots", slots)
    for name, t in (("bias_z", bias_z), ("bias_x", bias_x), ("state", state)):
        _need_f32(name, t)
    m, k = x.shape
    n = weight.shape[0] // 3
    if slots.numel() != m or bias_z.numel() != n or bias_x.numel() != n:
        raise KernelShapeError("linear_gru: one slot per row, one bias per column")
    if state.dim() != 2 or state.shape[1] != n or state.shape[0] < 2 or state.stride(1) != 1:
        raise KernelShapeError(f"linear_gru: state is [slots + 1, {n}] with unit inner stride, got {tuple(state.shape)}")
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    library.check(
        library.load().mi_gemm_skinny_gru_bf16(
            _ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias_z), _ptr(bias_x), _ptr(state), state.stride(0),
            _ptr(slots), state.shape[0] - 1, _ptr(out), out.stride(0), m, n, k, _stream(),
        )
    )
    return out


def linear_gelu_table(x: torch.Tensor, weight: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, first_col: int) -> torch.Tensor:
    """`gelu_tanh(x @ weight.T) * table[ids, first_col : first_col + N]`.  Few bfloat16 rows: one
    weight-streaming kernel with the activation and the gather in its last step; otherwise the
    product followed by `gated_table_rows`.  Both round the product to the element type first."""
    n = weight.shape[0]
    if (
        x.dtype == torch.bfloat16
        and weight.dtype == torch.bfloat16
        and table.dtype == torch.bfloat16
        and x.dim() == 2
        and weight.dim() == 2
        and x.shape[1] == weight.shape[1]
        and x.stride(1) == 1
        and weight.stride(1) == 1
        and skinny_gemm_takes(x.shape[0], x.shape[1], x.stride(0), weight.stride(0))
    ):
        _need_cuda(x, weight, table, ids)
        _need_contiguous("table", table)
        _need_contiguous("ids", ids)
        _need_int32("ids", ids)
        m, k = x.shape
        if table.dim() != 2 or ids.numel() != m or first_col < 0 or first_col + n > table.shape[1]:
            raise KernelShapeError(
                f"linear_gelu_table: columns {first_col}..{first_col + n} of a table with {table.shape[1]}, {ids.numel()} ids for {m} rows"
            )
        out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
        library.check(
            library.load().mi_gemm_skinny_gelu_table_bf16(
                _ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(table), table.stride(0), _ptr(ids),
                int(first_col), table.shape[0], _ptr(out), out.stride(0), m, n, k, _stream(),
            )
        )
        return out
    return gated_table_rows(linear(x, weight), table, ids, first_col)


# ----------------------------------------------------------------------------
# a layer whose sublayers share one norm and add their outputs together; a matrix-state
# recurrence behind a short convolution; attention over one latent row per token
# ----------------------------------------------------------------------------


@dataclasses.dataclass
class StreamUpdate:
    """An update of the float32 stream that has not been made yet:

        x += scale * (a + b + bias) + shift

    `a`, `b`: a layer's sublayer outputs [T, H] in the compute dtype (either may be None);
    `bias`, `shift`: float32 [H] or None.  A norm that knows it makes the update and its own
    statistics in one launch (`stream_update_norm`); anything else calls `finish()`, which
    returns the whole right-hand side as one float32 tensor to add."""

    a: torch.Tensor | None
    b: torch.Tensor | None = None
    bias: torch.Tensor | None = None
    shift: torch.Tensor | None = None
    scale: float = 1.0

    def shifted(self, shift: torch.Tensor) -> "StreamUpdate":
        """The same update with one more vector added to every row."""
        total = shift if self.shift is None else self.shift + shift
        return dataclasses.replace(self, shift=total)

    def finish(self) -> torch.Tensor:
        total = None
        for part in (self.a, self.b, self.bias):
            if part is not None:
                total = part.float() if total is None else total + part.float()
        if total is not None:
            total = total * self.scale
        if self.shift is not None:
            total = self.shift if total is None else total + self.shift
        if total is None:
            raise ValueError("an empty stream update")
        return total


def stream_update_norm(
    update: StreamUpdate | None, residual: torch.Tensor, weight: torch.Tensor | None, eps: float,
    rows: torch.Tensor | None = None,
) -> torch.Tensor | None:
    """Make `update` on the float32 stream in place (kept unless `rows`), then the RMS norm of the
    new rows times `weight` (compute dtype) -> [T, H] or [len(rows), H]; `weight=None`: the
    update alone."""
    update = update if update is not None else StreamUpdate(None)
    _need_cuda(update.a, update.b, update.bias, update.shift, residual, weight, rows)
    for name, t in (("residual", residual), ("weight", weight), ("rows", rows), ("bias", update.bias), ("shift", update.shift)):
        _need_contiguous(name, t)
    _need_int32("rows", rows)
    _need_f32("residual", residual)
    _need_f32("bias", update.bias)
    _need_f32("shift", update.shift)
    tokens, hidden = residual.shape
    dtype = weight.dtype if weight is not None else (update.a.dtype if update.a is not None else torch.float32)
    for name, t in (("a", update.a), ("b", update.b)):
        if t is not None and (t.dim() != 2 or tuple(t.shape) != (tokens, hidden) or t.stride(1) != 1 or t.dtype != dtype):
            raise KernelShapeError(f"stream update: {name} {tuple(t.shape)} {t.dtype} does not fit the stream {(tokens, hidden)} in {dtype}")
    for name, t in (("bias", update.bias), ("shift", update.shift), ("weight", weight)):
        if t is not None and t.numel() != hidden:
            raise KernelShapeError(f"stream update: {name} has {t.numel()} entries for {hidden} columns")
    if weight is None and rows is not None:
        raise KernelShapeError("stream update: a row list only goes with a norm")
    n_out = tokens if rows is None else rows.numel()
    out = torch.empty((n_out, hidden), dtype=dtype, device=residual.device) if weight is not None else None
    code = F32 if dtype == torch.float32 else BF16
    library.check(
        library.load().mi_stream_update_norm(
            code, _ptr(update.a), 0 if update.a is None else update.a.stride(0), _ptr(update.b),
            0 if update.b is None else update.b.stride(0), _ptr(update.bias), _ptr(update.shift), float(update.scale),
            _ptr(residual), _ptr(weight), _ptr(out), _ptr(rows), n_out, hidden, float(eps), _stream(),
        )
    )
    return out


def clamped_glu(gate_up: torch.Tensor, bias: torch.Tensor | None, limit: float, slope: float) -> torch.Tensor:
    """Rows [gate | up] (+ `bias`, float32 [2I]) -> `g * logistic(slope * g) * (u + 1)` with
    g = min(gate, limit), u = clamp(up, -limit, limit); returns [T, I]."""
    _need_cuda(gate_up, bias)
    _need_contiguous("bias", bias)
    _need_f32("bias", bias)
    if gate_up.dim() != 2 or gate_up.stride(1) != 1 or gate_up.shape[1] % 2 != 0:
        raise KernelShapeError(f"clamped_glu: rows hold [gate | up], got {tuple(gate_up.shape)} strides {gate_up.stride()}")
    tokens, inter = gate_up.shape[0], gate_up.shape[1] // 2
    if bias is not None and bias.numel() != 2 * inter:
        raise KernelShapeError(f"clamped_glu: the bias has {bias.numel()} entries for {2 * inter} columns")
    out = torch.empty((tokens, inter), dtype=gate_up.dtype, device=gate_up.device)
    library.check(
        library.load().mi_clamped_glu(
            _dtype_code(gate_up), _ptr(gate_up), gate_up.stride(0), _ptr(bias), _ptr(out), out.stride(0), tokens, inter,
            float(limit), float(slope), _stream(),
        )
    )
    return out


def linear_clamped_glu(x: torch.Tensor, gate_up_weight: torch.Tensor, bias: torch.Tensor, limit: float, slope: float) -> torch.Tensor:
    """`clamped_glu(x @ [gate; up].T, bias, limit, slope)`.  bfloat16 with at most 32 rows runs as ONE
    kernel (the weight-streaming product with biases, clamps and activation in its last step);
    otherwise the product and `clamped_glu` run in turn.  Both round the two products to the element
    type first and then do the same float32 arithmetic, so the results agree bit for bit."""
    rows, width = gate_up_weight.shape
    if rows % 2 or bias.numel() != rows:
        raise KernelShapeError(f"linear_clamped_glu: stacked weight of {rows} rows, bias of {bias.numel()}")
    if (
        x.dtype == torch.bfloat16
        and gate_up_weight.dtype == torch.bfloat16
        and x.dim() == 2
        and x.shape[1] == width
        and x.stride(1) == 1
        and gate_up_weight.stride(1) == 1
        and skinny_gemm_takes(x.shape[0], width, x.stride(0), gate_up_weight.stride(0), SKINNY_WIDE_MAX_ROWS)
    ):
        _need_cuda(x, gate_up_weight, bias)
        _need_contiguous("bias", bias)
        _need_f32("bias", bias)
        m, n = x.shape[0], rows // 2
        out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
        library.check(
            library.load().mi_gemm_skinny_clamped_glu_bf16(
                _ptr(x), x.stride(0), _ptr(gate_up_weight), gate_up_weight.stride(0), _ptr(bias), float(limit), float(slope),
                _ptr(out), out.stride(0), m, n, width, _stream(),
            )
        )
        return out
    return clamped_glu(linear(x, gate_up_weight), bias, limit, slope)


def linear_geglu(x: torch.Tensor, gate_up_weight: torch.Tensor) -> torch.Tensor:
    """`gelu_tanh(x @ gate.T) * (x @ up.T)` with `gate_up_weight` = [gate; up] stacked, [2I, K].  bfloat16
    with at most 32 rows runs as ONE kernel (the weight-streaming product with the activation in its
    last step); otherwise the product and `gated_mul` run in turn.  Both round the two products to the
    element type first and then do the same float32 arithmetic."""
    rows, width = gate_up_weight.shape
    if rows % 2:
        raise KernelShapeError(f"linear_geglu: stacked weight has an odd number of rows ({rows})")
    if (
        x.dtype == torch.bfloat16
        and gate_up_weight.dtype == torch.bfloat16
        and x.dim() == 2
        and x.shape[1] == width
        and x.stride(1) == 1
        and gate_up_weight.stride(1) == 1
        and skinny_gemm_takes(x.shape[0], width, x.stride(0), gate_up_weight.stride(0), SKINNY_WIDE_MAX_ROWS)
    ):
        _need_cuda(x, gate_up_weight)
        m, n = x.shape[0], rows // 2
        out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
        library.check(
            library.load().mi_gemm_skinny_geglu_bf16(
                _ptr(x), x.stride(0), _ptr(gate_up_weight), gate_up_weight.stride(0), _ptr(out), out.stride(0), m, n, width, _stream(),
            )
        )
        return out
    both = linear(x, gate_up_weight)
    return gated_mul(both[:, : rows // 2], both[:, rows // 2 :], "gelu_tanh")


def short_conv(
    x: torch.Tensor, channels: int, taps_weight: torch.Tensor, tail: torch.Tensor, cu_seqlens: torch.Tensor,
    slots: torch.Tensor, token_request: torch.Tensor, bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """A causal convolution over time per channel, then silu, on the first `channels` columns of
    `x` [T, >= channels]: `y[t, c] = silu(bias[c] + sum_j w[c, j] * x[t - (taps-1) + j, c])` within each
    request.  `tail` [slots + 1, taps - 1, channels] (compute dtype, rows may be strided) holds
    each request's last taps-1 inputs and is advanced in place; `taps_weight` is float32
    [channels, taps], last column the current token's."""
    _need_cuda(x, taps_weight, tail, cu_seqlens, slots, token_request, bias)
    for name, t in (("taps_weight", taps_weight), ("cu_seqlens", cu_seqlens), ("slots", slots), ("token_request", token_request),
                    ("bias", bias)):
        _need_contiguous(name, t)
    _need_f32("bias", bias)
    if bias is not None and bias.numel() != channels:
        raise KernelShapeError(f"short_conv: the bias has {bias.numel()} entries for {channels} channels")
    for name, t in (("cu_seqlens", cu_seqlens), ("slots", slots), ("token_request", token_request)):
        _need_int32(name, t)
    _need_f32("taps_weight", taps_weight)
    if x.dim() != 2 or x.stride(1) != 1 or x.shape[1] < channels:
        raise KernelShapeError(f"short_conv: x must be [T, >= {channels}] with unit inner stride, got {tuple(x.shape)}")
    if taps_weight.dim() != 2 or taps_weight.shape[0] != channels:
        raise KernelShapeError(f"short_conv: taps are [{channels}, taps], got {tuple(taps_weight.shape)}")
    taps = taps_weight.shape[1]
    tokens, requests = x.shape[0], slots.numel()
    if tail.dtype != x.dtype or tail.dim() != 3 or tuple(tail.shape[1:]) != (taps - 1, channels) or tail.shape[0] < 2:
        raise KernelShapeError(f"short_conv: the tail is {x.dtype} [slots + 1, {taps - 1}, {channels}], got {tail.dtype} {tuple(tail.shape)}")
    if taps > 1 and (tail.stride(2) != 1 or tail.stride(1) != channels):
        raise KernelShapeError(f"short_conv: a slot's tail must be packed, got strides {tail.stride()}")
    if cu_seqlens.numel() != requests + 1 or token_request.numel() != tokens:
        raise KernelShapeError("short_conv: one more boundary than requests, one request index per token")
    y = torch.empty((tokens, channels), dtype=x.dtype, device=x.device)
    library.check(
        library.load().mi_short_conv(
            _dtype_code(x), _ptr(x), x.stride(0), _ptr(taps_weight), _ptr(tail), tail.stride(0), _ptr(cu_seqlens), _ptr(slots),
            _ptr(token_request), _ptr(y), y.stride(0), tokens, requests, channels, taps, tail.shape[0] - 1, _ptr(bias), _stream(),
        )
    )
    return y


def delta_state_shape(heads: int, dim: int, vdim: int) -> tuple[int, int, int]:
    """How `gated_delta` lays a request's state out: per head S transposed, [vdim][padded dim].
    A column is kept by 16 neighbouring lanes with 4, 8 or 16 rows each: the padded dim is their
    product (the kernel checks it)."""
    return (heads, vdim, 64 if dim <= 64 else (128 if dim <= 128 else 256))


def gated_delta(
    qkv: torch.Tensor, proj: torch.Tensor, col_b: int, col_a: int, col_g: int, a_log: torch.Tensor, dt_bias: torch.Tensor,
    norm_weight: torch.Tensor, state: torch.Tensor, cu_seqlens: torch.Tensor, slots: torch.Tensor, *, heads: int,
    kv_heads: int, dim: int, vdim: int, eps: float,
) -> torch.Tensor:
    """The gated delta rule over the rows of a step.  `qkv` [T, 2*kv_heads*dim + heads*vdim]: the
    convolved q | k | v; `proj` [T, ...]: the rows that hold, from columns `col_b`, `col_a`
    (heads each) and `col_g` (heads*vdim) on, the projections of the write gate, the decay and
    the output gate.  `state` float32 [slots + 1, *delta_state_shape(...)] is advanced in
    place.  Returns `rms_norm(S^T q) * norm_weight * silu(g)` [T, heads*vdim]."""
    _need_cuda(qkv, proj, a_log, dt_bias, norm_weight, state, cu_seqlens, slots)
    for name, t in (("a_log", a_log), ("dt_bias", dt_bias), ("norm_weight", norm_weight), ("cu_seqlens", cu_seqlens), ("slots", slots)):
        _need_contiguous(name, t)
    for name, t in (("a_log", a_log), ("dt_bias", dt_bias), ("norm_weight", norm_weight), ("state", state)):
        _need_f32(name, t)
    _need_int32("cu_seqlens", cu_seqlens)
    _need_int32("slots", slots)
    width = 2 * kv_heads * dim + heads * vdim
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < width:
        raise KernelShapeError(f"gated_delta: qkv must be [T, >= {width}] with unit inner stride, got {tuple(qkv.shape)}")
    if proj.dim() != 2 or proj.stride(1) != 1 or proj.shape[0] != qkv.shape[0] or proj.dtype != qkv.dtype:
        raise KernelShapeError("gated_delta: the gates' projections are rows of the same step and dtype")
    if max(col_b + heads, col_a + heads, col_g + heads * vdim) > proj.shape[1]:
        raise KernelShapeError("gated_delta: the gates' columns lie outside the projections' rows")
    if a_log.numel() != heads or dt_bias.numel() != heads or norm_weight.numel() != vdim:
        raise KernelShapeError("gated_delta: one decay rate and one step bias per head, one norm weight per value column")
    shape = delta_state_shape(heads, dim, vdim)
    if state.dim() != 4 or tuple(state.shape[1:]) != shape or state.shape[0] < 2 or not state[0].is_contiguous():
        raise KernelShapeError(f"gated_delta: the state is float32 [slots + 1, {shape}] with packed slots, got {tuple(state.shape)}")
    requests = slots.numel()
    if cu_seqlens.numel() != requests + 1:
        raise KernelShapeError("gated_delta: one more boundary than requests")
    out = torch.empty((qkv.shape[0], heads * vdim), dtype=qkv.dtype, device=qkv.device)
    readout = torch.empty((qkv.shape[0], heads * vdim), dtype=torch.float32, device=qkv.device)  # S^T q before its norm
    library.check(
        library.load().mi_gated_delta(
            _dtype_code(qkv), _ptr(qkv), qkv.stride(0), _ptr(proj), proj.stride(0), int(col_b), int(col_a), int(col_g),
            _ptr(a_log), _ptr(dt_bias), _ptr(norm_weight), _ptr(state), state.stride(0), _ptr(cu_seqlens), _ptr(slots),
            _ptr(readout), _ptr(out), out.stride(0), qkv.shape[0], requests, heads, kv_heads, dim, vdim, shape[2], float(eps),
            state.shape[0] - 1, _stream(),
        )
    )
    return out


def latent_prepare(
    proj: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, norm_weight: torch.Tensor, slot_mapping: torch.Tensor | None,
    k_pages: torch.Tensor | None, queries: torch.Tensor | None, *, heads: int, q_head_width: int, q_rot_at: int, c_col: int,
    rank: int, rot: int, eps: float, latent_out: torch.Tensor | None = None, down: torch.Tensor | None = None,
) -> None:
    """What a latent attention layer does between its projections and its attention.  `proj`
    [T, ...] holds the query heads (`q_head_width` columns each from column 0 on, the part to
    rotate `rot` wide from `q_rot_at` inside a head) and from `c_col` on [x_c (rank) | x_r (rot)].
    Writes `[rms_norm(x_c) * norm_weight | rotated x_r]` into the token's slot of `k_pages`
    ([num_pages, 1, page_size, rank + rot]; nothing with `slot_mapping=None`) and each head's
    rotated query part into the last `rot` columns of its [rank + rot] wide piece of `queries`
    (`queries=None`: not wanted).  `latent_out` [T, rank]: a copy of the normed latents, if wanted.
    `down` [T, ...]: rows of their own that hold [x_c | x_r] from `c_col` on, where the queries come
    from a product of their own (`proj` then holds the query heads alone)."""
    _need_cuda(proj, cos, sin, norm_weight, slot_mapping, k_pages, queries, latent_out, down)
    if down is not None and (down.dim() != 2 or down.stride(1) != 1 or down.dtype != proj.dtype or down.shape[0] != proj.shape[0]
                             or down.shape[1] < c_col + rank + rot):
        raise KernelShapeError(f"latent_prepare: the latent rows must be {proj.dtype} [{proj.shape[0]}, >= {c_col + rank + rot}]")
    _need_contiguous("latent_out", latent_out)
    if latent_out is not None and (latent_out.dtype != proj.dtype or tuple(latent_out.shape) != (proj.shape[0], rank)):
        raise KernelShapeError(f"latent_prepare: latent_out is {proj.dtype} [{proj.shape[0]}, {rank}], got {latent_out.dtype} {tuple(latent_out.shape)}")
    for name, t in (("cos", cos), ("sin", sin), ("norm_weight", norm_weight), ("slot_mapping", slot_mapping), ("k_pages", k_pages)):
        _need_contiguous(name, t)
    _need_int32("slot_mapping", slot_mapping)
    _need_f32("norm_weight", norm_weight)
    tokens = proj.shape[0]
    if proj.dim() != 2 or proj.stride(1) != 1 or proj.shape[1] < max(heads * q_head_width, 0 if down is not None else c_col + rank + rot):
        raise KernelShapeError(f"latent_prepare: the projections' rows are too short, got {tuple(proj.shape)}")
    if queries is not None and (queries.dtype != proj.dtype or queries.dim() != 2 or queries.stride(1) != 1
                                or tuple(queries.shape) != (tokens, heads * (rank + rot))):
        raise KernelShapeError(f"latent_prepare: queries are {proj.dtype} [{tokens}, {heads * (rank + rot)}], got {queries.dtype} {tuple(queries.shape)}")
    if cos.dtype != torch.float32 or tuple(cos.shape) != (tokens, rot // 2) or sin.shape != cos.shape or sin.dtype != torch.float32:
        raise KernelShapeError(f"latent_prepare: cos/sin must be float32 [{tokens}, {rot // 2}], got {tuple(cos.shape)} {cos.dtype}")
    if norm_weight.numel() != rank:
        raise KernelShapeError(f"latent_prepare: the norm weight has {norm_weight.numel()} entries for a latent of {rank}")
    if slot_mapping is not None:
        if k_pages is None or k_pages.dtype != proj.dtype or k_pages.dim() != 4 or k_pages.shape[1] != 1 or k_pages.shape[3] != rank + rot:
            raise KernelShapeError(f"latent_prepare: key pages must be {proj.dtype} [num_pages, 1, page_size, {rank + rot}]")
        if slot_mapping.numel() != tokens:
            raise KernelShapeError(f"slot_mapping has {slot_mapping.numel()} entries for {tokens} tokens")
    library.check(
        library.load().mi_latent_prepare(
            _dtype_code(proj), _ptr(proj), proj.stride(0), 0, int(q_head_width), int(q_rot_at), int(c_col), _ptr(cos), _ptr(sin),
            _ptr(norm_weight), _ptr(slot_mapping), _ptr(k_pages) if slot_mapping is not None else None, _ptr(queries),
            0 if queries is None else queries.stride(0), _ptr(latent_out), tokens, heads, rank, rot, float(eps),
            _ptr(down), 0 if down is None else down.stride(0), _stream(),
        )
    )


def latent_expand(
    proj: torch.Tensor, k_up: torch.Tensor, v_up: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, *, heads: int,
    dim: int, rot: int, vdim: int, r_col: int, down: torch.Tensor | None = None,
) -> torch.Tensor:
    """One row [q | k | v] per token with `heads` heads of D = dim + rot columns each, from a latent
    attention layer's projections (`proj`: query heads [plain (dim) | to rotate (rot)] from column 0
    on, the shared part to rotate from `r_col` on), the keys' plain parts `k_up` [T, heads*dim] and the
    values `v_up` [T, heads*vdim] (padded with zeros to D): what the paged attention kernels take."""
    _need_cuda(proj, k_up, v_up, cos, sin)
    for name, t in (("proj", proj), ("k_up", k_up), ("v_up", v_up)):
        if t.dim() != 2 or t.stride(1) != 1 or t.dtype != proj.dtype or t.shape[0] != proj.shape[0]:
            raise KernelShapeError(f"latent_expand: {name} must be rows of the step in {proj.dtype} with unit inner stride")
    _need_contiguous("cos", cos)
    _need_contiguous("sin", sin)
    tokens, width = proj.shape[0], dim + rot
    if cos.dtype != torch.float32 or tuple(cos.shape) != (tokens, rot // 2) or sin.shape != cos.shape or sin.dtype != torch.float32:
        raise KernelShapeError(f"latent_expand: cos/sin must be float32 [{tokens}, {rot // 2}]")
    if down is not None and (down.dim() != 2 or down.stride(1) != 1 or down.dtype != proj.dtype or down.shape[0] != tokens
                             or down.shape[1] < r_col + rot):
        raise KernelShapeError("latent_expand: the rows that hold the shared part do not fit")
    if k_up.shape[1] != heads * dim or v_up.shape[1] != heads * vdim or vdim > width or proj.shape[1] < max(
            heads * width, 0 if down is not None else r_col + rot):
        raise KernelShapeError("latent_expand: the projections do not hold what the sizes say")
    qkv = torch.empty((tokens, 3 * heads * width), dtype=proj.dtype, device=proj.device)
    library.check(
        library.load().mi_latent_expand(
            _dtype_code(proj), _ptr(proj), proj.stride(0), width, dim, int(r_col), _ptr(k_up), k_up.stride(0), _ptr(v_up),
            v_up.stride(0), _ptr(cos), _ptr(sin), _ptr(qkv), qkv.stride(0), tokens, heads, dim, rot, vdim,
            _ptr(down), 0 if down is None else down.stride(0), _stream(),
        )
    )
    return qkv


def linear_per_head(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor) -> None:
    """`out[:, h, :] = x[:, h, :] @ weight[h].T` for every head h: x [T, heads, K], weight
    [heads, N, K], out [T, heads, N]; x and out may be views into wider rows (unit inner
    stride).  float32: the true-float32 product, head by head; bfloat16: one batched product of
    the vendor library (the weight-streaming product has no batched form; head by head it costs a
    launch a head, which at few rows is all a step's time)."""
    _need_cuda(x, weight, out)
    if x.dim() != 3 or weight.dim() != 3 or out.dim() != 3 or x.stride(2) != 1 or out.stride(2) != 1 or weight.stride(2) != 1:
        raise KernelShapeError("linear_per_head: x [T, heads, K], weight [heads, N, K], out [T, heads, N], unit inner strides")
    tokens, heads, k = x.shape
    n = weight.shape[1]
    if tuple(weight.shape) != (heads, n, k) or tuple(out.shape) != (tokens, heads, n) or not (x.dtype == weight.dtype == out.dtype):
        raise KernelShapeError(f"linear_per_head: shapes {tuple(x.shape)}, {tuple(weight.shape)}, {tuple(out.shape)} do not fit")
    if tokens == 0:
        return
    lib = library.load()
    if x.dtype == torch.float32:
        for h in range(heads):
            library.check(lib.mi_gemm_f32(_ptr(x[:, h]), x.stride(0), _ptr(weight[h]), weight.stride(1), _ptr(out[:, h]),
                                          out.stride(0), tokens, n, k, _stream()))
        return
    torch.bmm(x.transpose(0, 1), weight.transpose(1, 2), out=out.transpose(0, 1))


def sample(
    logits: torch.Tensor,
    temperature: torch.Tensor,
    top_k: torch.Tensor,
    top_p: torch.Tensor,
    seed_lo: torch.Tensor,
    seed_hi: torch.Tensor,
    draw_index: torch.Tensor,
) -> torch.Tensor:
    """One token id per row of `logits` [B, V]; per-row settings are device tensors of length B.

    `temperature` and `top_p` are float32, `top_k` int32, `seed_lo`, `seed_hi` and
    `draw_index` int32 holding unsigned 32-bit patterns.
    """
    _need_cuda(logits, temperature, top_k, top_p, seed_lo, seed_hi, draw_index)
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelShapeError("logits must be [rows, vocab] with unit inner stride")
    rows, vocab = logits.shape
    for name, t, dt in (
        ("temperature", temperature, torch.float32),
        ("top_k", top_k, torch.int32),
        ("top_p", top_p, torch.float32),
        ("seed_lo", seed_lo, torch.int32),
        ("seed_hi", seed_hi, torch.int32),
        ("draw_index", draw_index, torch.int32),
    ):
        _need_contiguous(name, t)
        if t.dtype != dt or t.numel() != rows:
            raise KernelShapeError(f"{name} must be {dt} with {rows} entries, got {t.dtype} x {t.numel()}")
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    lib = library.load()
    library.check(
        lib.mi_sample(
            _dtype_code(logits), _ptr(logits), logits.stride(0), rows, vocab, _ptr(temperature),
            _ptr(top_k), _ptr(top_p), _ptr(seed_lo), _ptr(seed_hi), _ptr(draw_index), _ptr(out),
            _stream(),
        )
    )
    return out


def sample_slots(logits: torch.Tensor, slots: torch.Tensor, slot_table: torch.Tensor) -> torch.Tensor:
    """One token id per row of `logits` [B, V], each row's settings (temperature, top_k, top_p,
    seed, draw index) read from row `slots[b]` of `slot_table` [slots, 8] int32; the draw
    index of every sampled slot is advanced by one on the device.  No slot may appear in two
    rows; a row whose slot id lies outside the table (the -1 of a padding row) is sampled
    greedily and writes nothing."""
    _need_cuda(logits, slots, slot_table)
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelShapeError("logits must be [rows, vocab] with unit inner stride")
    rows, vocab = logits.shape
    for name, t in (("slots", slots), ("slot_table", slot_table)):
        _need_contiguous(name, t)
        _need_int32(name, t)
    if slots.numel() != rows or slot_table.dim() != 2 or slot_table.shape[1] != SLOT_WORDS:
        raise KernelShapeError(f"sample_slots: one slot id per row and a table [slots, {SLOT_WORDS}]")
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    lib = library.load()
    library.check(
        lib.mi_sample_slots(
            _dtype_code(logits), _ptr(logits), logits.stride(0), rows, vocab, _ptr(slots), _ptr(slot_table),
            slot_table.shape[0], _ptr(out), _stream(),
        )
    )
    return out


# ----------------------------------------------------------------------------
# a stream kept in several copies; recurrences with a decaying matrix state; heads normed one by one
# ----------------------------------------------------------------------------

MAX_STREAM_COPIES = 8


def embed_norm_streams(table: torch.Tensor, ids: torch.Tensor, weight: torch.Tensor, copies: int, eps: float) -> torch.Tensor:
    """`x = table[ids]`, divided by its root mean square (eps inside the root), times `weight`
    (float32 [H], the factor itself), written `copies` times: float32 [T, copies, H]."""
    _need_cuda(table, ids, weight)
    for name, t in (("table", table), ("ids", ids), ("weight", weight)):
        _need_contiguous(name, t)
    _need_int32("ids", ids)
    _need_f32("weight", weight)
    vocab, hidden = table.shape
    if weight.numel() != hidden or not 1 <= copies <= MAX_STREAM_COPIES:
        raise KernelShapeError(f"embed_norm_streams: weight of {weight.numel()} for {hidden} columns, {copies} copies (1..{MAX_STREAM_COPIES})")
    out = torch.empty((ids.numel(), copies, hidden), dtype=torch.float32, device=table.device)
    library.check(
        library.load().mi_embed_norm_streams(
            _dtype_code(table), _ptr(table), _ptr(ids), _ptr(weight), _ptr(out), ids.numel(), hidden, vocab, copies, float(eps),
            _stream(),
        )
    )
    return out


@dataclasses.dataclass
class StreamsWrite:
    """A sublayer's write into a stream kept in S copies that has not been made yet:

        y = scale_a * a + scale_b * b;      x_t <- sum_s mix[s, t] * x_s + out[t] * y      (all copies at once)

    `a`, `b`: sublayer outputs [T, H] in the compute dtype (`b` may be None); `mix` float32 [S, S]
    indexed [from, to], `out` float32 [S].  A norm that knows it makes the write together with
    the next read and its own statistics in one launch (`streams_update_norm`); `apply(streams)`
    makes the write alone."""

    a: torch.Tensor
    mix: torch.Tensor
    out: torch.Tensor
    b: torch.Tensor | None = None
    scale_a: float = 1.0
    scale_b: float = 1.0

    def apply(self, streams: torch.Tensor) -> None:
        streams_update_norm(self, streams, None, None, 0.0, self.a.dtype)


def streams_update_norm(
    write: StreamsWrite | None, streams: torch.Tensor, read: torch.Tensor | None, weight: torch.Tensor | None, eps: float,
    dtype: torch.dtype, rows: torch.Tensor | None = None,
) -> torch.Tensor | None:
    """Make `write` on the float32 copies [T, S, H] in place (kept unless `rows`), then read them
    as `u = sum_t read[t] * x_t` (`read` float32 [S]; None: the plain sum) and return
    `u / rms(u) * weight` (`weight` float32 [H], the factor itself) in `dtype`: [T, H] or
    [len(rows), H].  `weight=None`: the write alone."""
    tensors = (streams, read, weight, rows) + ((write.a, write.b, write.mix, write.out) if write is not None else ())
    _need_cuda(*tensors)
    for name, t in (("streams", streams), ("read", read), ("weight", weight), ("rows", rows)):
        _need_contiguous(name, t)
    _need_int32("rows", rows)
    for name, t in (("streams", streams), ("read", read), ("weight", weight)):
        _need_f32(name, t)
    if streams.dim() != 3 or not 1 <= streams.shape[1] <= MAX_STREAM_COPIES:
        raise KernelShapeError(f"streams are float32 [T, copies <= {MAX_STREAM_COPIES}, H], got {tuple(streams.shape)}")
    tokens, copies, hidden = streams.shape
    if read is not None and read.numel() != copies:
        raise KernelShapeError(f"the read vector has {read.numel()} entries for {copies} copies")
    if weight is not None and weight.numel() != hidden:
        raise KernelShapeError(f"the norm weight has {weight.numel()} entries for {hidden} columns")
    if weight is None and rows is not None:
        raise KernelShapeError("a row list only goes with a norm")
    a = b = mix = out_vec = None
    scale_a = scale_b = 1.0
    if write is not None:
        a, b, mix, out_vec, scale_a, scale_b = write.a, write.b, write.mix, write.out, write.scale_a, write.scale_b
        _need_f32("mix", mix)
        _need_f32("out", out_vec)
        _need_contiguous("mix", mix)
        _need_contiguous("out", out_vec)
        if tuple(mix.shape) != (copies, copies) or out_vec.numel() != copies:
            raise KernelShapeError(f"a write into {copies} copies needs mix [{copies}, {copies}] and out [{copies}]")
        for name, t in (("a", a), ("b", b)):
            if t is not None and (t.dim() != 2 or tuple(t.shape) != (tokens, hidden) or t.stride(1) != 1 or t.dtype != dtype):
                raise KernelShapeError(f"streams write: {name} {tuple(t.shape)} {t.dtype} does not fit {(tokens, hidden)} in {dtype}")
    n_out = tokens if rows is None else rows.numel()
    result = torch.empty((n_out, hidden), dtype=dtype, device=streams.device) if weight is not None else None
    library.check(
        library.load().mi_streams_update_norm(
            F32 if dtype == torch.float32 else BF16, _ptr(a), 0 if a is None else a.stride(0), _ptr(b),
            0 if b is None else b.stride(0), float(scale_a), float(scale_b), _ptr(mix), _ptr(out_vec), _ptr(read), _ptr(weight),
            _ptr(streams), _ptr(result), _ptr(rows), n_out, hidden, copies, float(eps), _stream(),
        )
    )
    return result


def decay_state_shape(heads: int, dim: int, vdim: int) -> tuple[int, int, int]:
    """How `decay_scan` lays a request's state out: per head S transposed, [vdim][padded dim]."""
    if dim > 256:
        raise KernelShapeError(f"decay_scan takes key widths up to 256, got {dim}")
    pad = 16 if dim <= 16 else (32 if dim <= 32 else (64 if dim <= 64 else (128 if dim <= 128 else 256)))
    return (heads, vdim, pad)


def decay_scan(
    q: torch.Tensor, q_col: int, k: torch.Tensor, k_col: int, v: torch.Tensor, v_col: int, gate: torch.Tensor, gate_col: int,
    gate_bias: torch.Tensor, state: torch.Tensor, cu_seqlens: torch.Tensor, slots: torch.Tensor, *, heads: int, groups: int,
    dim: int, vdim: int, per_head: bool, rate: torch.Tensor | None = None, skip: torch.Tensor | None = None,
    inv_tau: float = 1.0, q_scale: float = 1.0,
) -> torch.Tensor:
    """The recurrence `S <- diag(a) S + k v^T; o = S^T q` over the rows of a step, per request and
    head, float32 state [slots + 1, *decay_state_shape(...)] advanced in place; returns the
    read-outs float32 [T, heads*vdim].

    `q`, `k`: rows that hold `groups` heads of `dim` from `q_col` / `k_col` on (head h reads
    group h // (heads // groups)); `v`: rows that hold `heads` heads of `vdim` from `v_col` on.
    `per_head=False`: `gate` rows hold heads*dim logits z from `gate_col` on and
    `a = logistic(z + gate_bias) ** inv_tau`, q enters times `q_scale`.  `per_head=True`: `gate`
    rows hold `heads` raw step sizes, `dt = softplus(raw + gate_bias)`, `a = exp(-exp(rate) * dt)`,
    v enters times dt and the read-out gets `skip[h] * v` added."""
    _need_cuda(q, k, v, gate, gate_bias, state, cu_seqlens, slots, rate, skip)
    for name, t in (("gate_bias", gate_bias), ("cu_seqlens", cu_seqlens), ("slots", slots), ("rate", rate), ("skip", skip)):
        _need_contiguous(name, t)
    for name, t in (("gate_bias", gate_bias), ("rate", rate), ("skip", skip), ("state", state)):
        _need_f32(name, t)
    _need_int32("cu_seqlens", cu_seqlens)
    _need_int32("slots", slots)
    tokens = q.shape[0]
    for name, t in (("q", q), ("k", k), ("v", v), ("gate", gate)):
        if t.dim() != 2 or t.stride(1) != 1 or t.shape[0] != tokens or t.dtype != q.dtype:
            raise KernelShapeError(f"decay_scan: {name} must be rows of the same step and dtype with unit inner stride")
    if q.shape[1] < q_col + groups * dim or k.shape[1] < k_col + groups * dim or v.shape[1] < v_col + heads * vdim:
        raise KernelShapeError("decay_scan: the q, k or v columns lie outside their rows")
    gate_width = heads if per_head else heads * dim
    if gate.shape[1] < gate_col + gate_width or gate_bias.numel() != gate_width:
        raise KernelShapeError(f"decay_scan: the gates need {gate_width} columns and as many biases")
    if per_head and (rate is None or rate.numel() != heads or (skip is not None and skip.numel() != heads)):
        raise KernelShapeError("decay_scan: one rate (and one skip weight) per head")
    shape = decay_state_shape(heads, dim, vdim)
    if state.dim() != 4 or tuple(state.shape[1:]) != shape or state.shape[0] < 2 or not state[0].is_contiguous():
        raise KernelShapeError(f"decay_scan: the state is float32 [slots + 1, {shape}] with packed slots, got {tuple(state.shape)}")
    requests = slots.numel()
    if cu_seqlens.numel() != requests + 1:
        raise KernelShapeError("decay_scan: one more boundary than requests")
    out = torch.empty((tokens, heads * vdim), dtype=torch.float32, device=q.device)
    library.check(
        library.load().mi_decay_scan(
            _dtype_code(q), int(per_head), _ptr(q), q.stride(0), int(q_col), _ptr(k), k.stride(0), int(k_col), _ptr(v),
            v.stride(0), int(v_col), _ptr(gate), gate.stride(0), int(gate_col), _ptr(gate_bias), _ptr(rate), _ptr(skip),
            float(inv_tau), float(q_scale), _ptr(state), state.stride(0), _ptr(cu_seqlens), _ptr(slots), state.shape[0] - 1,
            _ptr(out), tokens, requests, heads, groups, dim, vdim, _stream(),
        )
    )
    return out


def readout_gate_norm(
    readout: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, *, group_width: int, gate_first: bool, eps: float,
) -> torch.Tensor:
    """What follows a recurrence's read-outs (float32 [T, W]): an RMS norm over groups of
    `group_width` columns times `weight` (float32; column c takes `weight[c % len(weight)]`) and
    the gate `silu(gate)` ([T, W] in the compute dtype, rows may be strided).  `gate_first`:
    `norm(o * silu(g)) * w`, else `norm(o) * w * silu(g)`.  Returns [T, W] in the gate's dtype."""
    _need_cuda(readout, gate, weight)
    _need_contiguous("readout", readout)
    _need_contiguous("weight", weight)
    _need_f32("readout", readout)
    _need_f32("weight", weight)
    tokens, width = readout.shape
    if gate.dim() != 2 or gate.stride(1) != 1 or gate.shape[0] != tokens or gate.shape[1] < width:
        raise KernelShapeError(f"readout_gate_norm: the gate must be [T, >= {width}] with unit inner stride")
    if width % group_width != 0 or width % weight.numel() != 0:
        raise KernelShapeError(f"readout_gate_norm: {width} columns in groups of {group_width} with a weight of {weight.numel()}")
    out = torch.empty((tokens, width), dtype=gate.dtype, device=gate.device)
    library.check(
        library.load().mi_readout_gate_norm(
            _dtype_code(gate), _ptr(readout), _ptr(gate), gate.stride(0), _ptr(weight), weight.numel(), _ptr(out), out.stride(0),
            tokens, width, int(group_width), int(gate_first), float(eps), _stream(),
        )
    )
    return out


def head_norm_rope_kv_write(
    qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, slot_mapping: torch.Tensor | None, k_pages: torch.Tensor | None,
    v_pages: torch.Tensor | None, q_weight: torch.Tensor | None, k_weight: torch.Tensor | None, eps: float, *, q_heads: int,
    kv_heads: int, head_dim: int, rotary_dim: int, interleaved: bool = False, v_transposed: bool = False,
    v_head_dim: int | None = None,
) -> None:
    """`rope_kv_write` with every query and key head first divided by its own root mean square
    over the head and multiplied by `q_weight` / `k_weight` (float32 [head_dim], shared by the
    heads; None: that side is not normed)."""
    _need_cuda(qkv, cos, sin, slot_mapping, k_pages, v_pages, q_weight, k_weight)
    for name, t in (("cos", cos), ("sin", sin), ("slot_mapping", slot_mapping), ("k_pages", k_pages), ("v_pages", v_pages),
                    ("q_weight", q_weight), ("k_weight", k_weight)):
        _need_contiguous(name, t)
    _need_int32("slot_mapping", slot_mapping)
    _need_f32("q_weight", q_weight)
    _need_f32("k_weight", k_weight)
    if qkv.dim() != 2 or qkv.stride(1) != 1:
        raise KernelShapeError(f"qkv must be [T, width] with unit inner stride, got {qkv.stride()}")
    tokens = qkv.shape[0]
    v_dim = head_dim if v_head_dim is None else int(v_head_dim)
    if qkv.shape[1] < (q_heads + kv_heads) * head_dim + kv_heads * v_dim:
        raise KernelShapeError("qkv rows hold fewer values than the q, k and v heads need")
    if cos.shape != (tokens, rotary_dim // 2) or sin.shape != cos.shape or cos.dtype != torch.float32 or sin.dtype != torch.float32:
        raise KernelShapeError(f"cos/sin must be float32 [{tokens}, {rotary_dim // 2}], got {tuple(cos.shape)} {cos.dtype}")
    for name, t in (("q_weight", q_weight), ("k_weight", k_weight)):
        if t is not None and t.numel() != head_dim:
            raise KernelShapeError(f"{name} has {t.numel()} entries for heads of {head_dim}")
    page_size = num_pages = 0
    if kv_heads > 0 and slot_mapping is not None:
        if k_pages is None or v_pages is None:
            raise KernelShapeError("writing keys and values needs k_pages and v_pages")
        if k_pages.dtype != qkv.dtype or v_pages.dtype != qkv.dtype:
            raise KernelShapeError(f"pages are {k_pages.dtype}, activations {qkv.dtype}")
        if k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != head_dim:
            raise KernelShapeError(f"pages must be [num_pages, {kv_heads}, page_size, {head_dim}], got {tuple(k_pages.shape)}")
        _check_v_pages(k_pages, v_pages, v_transposed, v_dim)
        if slot_mapping.numel() != tokens:
            raise KernelShapeError(f"slot_mapping has {slot_mapping.numel()} entries for {tokens} tokens")
        num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
    library.check(
        library.load().mi_head_norm_rope_kv_write(
            _dtype_code(qkv), _ptr(qkv), qkv.stride(0), _ptr(cos), _ptr(sin), _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages),
            _ptr(q_weight), _ptr(k_weight), float(eps), tokens, q_heads, kv_heads, head_dim, rotary_dim, int(interleaved),
            page_size, num_pages, int(v_transposed), v_dim, _stream(),
        )
    )


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "logistic": 2}


def gated_mul(a: torch.Tensor, b: torch.Tensor, activation: str) -> torch.Tensor:
    """`act(a) * b` elementwise for [T, W] column ranges of rows (rows may be strided):
    `silu`, `gelu_tanh` (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))) or `logistic`."""
    if activation not in GATE_ACTIVATIONS:
        raise KernelShapeError(f"gated_mul: activation {activation!r}; built: {sorted(GATE_ACTIVATIONS)}")
    _need_cuda(a, b)
    if a.dim() != 2 or a.shape != b.shape or a.stride(1) != 1 or b.stride(1) != 1 or a.dtype != b.dtype:
        raise KernelShapeError(f"gated_mul: two [T, W] ranges of one dtype with unit inner stride, got {tuple(a.shape)} {tuple(b.shape)}")
    tokens, width = a.shape
    out = torch.empty((tokens, width), dtype=a.dtype, device=a.device)
    library.check(
        library.load().mi_gated_mul(
            _dtype_code(a), GATE_ACTIVATIONS[activation], _ptr(a), a.stride(0), _ptr(b), b.stride(0), _ptr(out), out.stride(0),
            tokens, width, _stream(),
        )
    )
    return out


@dataclasses.dataclass
class WeightedSum:
    """`scale_a * a + scale_b * b` of two sublayer outputs [T, H] in the compute dtype, not made
    yet: a stream write that knows it (`StreamsWrite`) makes it on its way; anything else calls
    `finish()`."""

    a: torch.Tensor
    b: torch.Tensor
    scale_a: float = 1.0
    scale_b: float = 1.0

    def finish(self) -> torch.Tensor:
        return (self.scale_a * self.a.float() + self.scale_b * self.b.float()).to(self.a.dtype)


# ----------------------------------------------------------------------------
# a stack normed behind the residual sum; an embedding with a hashed pair table
# ----------------------------------------------------------------------------


def embed_pair_hash(
    table: torch.Tensor, pairs: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor, token_request: torch.Tensor,
    cu_seqlens_q: torch.Tensor, state_slots: torch.Tensor, last_token: torch.Tensor, *, mul_prev: int, mul_cur: int,
    want_cast: bool = False,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """`float32(table[ids]) + pairs[row]`, `row = (prev * mul_prev + id * mul_cur) mod buckets` where
    `prev` is the token before in the same sequence, and `buckets` (the last row of `pairs`
    [buckets + 1, H]) for a sequence's first token.  The token before a request's first token of
    this step is read from `last_token` [slots + 1, >= 1] (int32, one row a state slot, the last row
    nobody's) at the request's slot, and the request's last token of the step is left there.
    Returns the float32 stream [T, H] and, with `want_cast`, the same rows in the table's dtype."""
    _need_cuda(table, pairs, ids, positions, token_request, cu_seqlens_q, state_slots, last_token)
    for name, t in (("table", table), ("pairs", pairs), ("ids", ids), ("positions", positions), ("token_request", token_request),
                    ("cu_seqlens_q", cu_seqlens_q), ("state_slots", state_slots)):
        _need_contiguous(name, t)
    for name, t in (("ids", ids), ("positions", positions), ("token_request", token_request), ("cu_seqlens_q", cu_seqlens_q),
                    ("state_slots", state_slots), ("last_token", last_token)):
        _need_int32(name, t)
    vocab, hidden = table.shape
    if pairs.dim() != 2 or pairs.shape[1] != hidden or pairs.shape[0] < 2 or pairs.dtype != table.dtype:
        raise KernelShapeError(f"embed_pair_hash: the pair table must be {table.dtype} [buckets + 1, {hidden}], got {pairs.dtype} {tuple(pairs.shape)}")
    tokens = ids.numel()
    if positions.numel() != tokens or token_request.numel() != tokens:
        raise KernelShapeError("embed_pair_hash: one position and one request per token id")
    if state_slots.numel() + 1 != cu_seqlens_q.numel():
        raise KernelShapeError("embed_pair_hash: one state slot per request")
    if last_token.dim() < 1 or last_token.shape[0] < 2:
        raise KernelShapeError("embed_pair_hash: the state rows are [slots + 1, ...]")
    out = torch.empty((tokens, hidden), dtype=torch.float32, device=table.device)
    cast = torch.empty((tokens, hidden), dtype=table.dtype, device=table.device) if want_cast else None
    library.check(
        library.load().mi_embed_pair_hash(
            _dtype_code(table), _ptr(table), _ptr(pairs), _ptr(ids), _ptr(positions), _ptr(token_request), _ptr(cu_seqlens_q),
            _ptr(state_slots), _ptr(last_token), last_token.stride(0), last_token.shape[0] - 1, _ptr(out), _ptr(cast), tokens,
            hidden, vocab, pairs.shape[0] - 1, int(mul_prev), int(mul_cur), _stream(),
        )
    )
    return out, cast


def scale_add_norm(
    residual: torch.Tensor, y: torch.Tensor | None, scale: torch.Tensor | None, factor: torch.Tensor, alpha: float,
    eps: float, dtype: torch.dtype, rows: torch.Tensor | None = None, want_cast: bool = True,
) -> torch.Tensor | None:
    """The norm behind the sum: `x <- rms_norm(alpha * x + scale * y) * factor` row by row, in place
    on the float32 stream `residual` [T, H] (`scale`, `factor` float32 [H]; without `scale` the sum
    is `alpha * x + y`; without `y` the row is normed as it is).  With `want_cast` the new rows are
    returned in `dtype` as well.  With `rows` (int32) only those rows are normed, the stream stays
    as it was and the normed rows come back [len(rows), H]."""
    _need_cuda(residual, y, scale, factor, rows)
    for name, t in (("residual", residual), ("scale", scale), ("factor", factor), ("rows", rows)):
        _need_contiguous(name, t)
    _need_f32("residual", residual)
    _need_f32("scale", scale)
    _need_f32("factor", factor)
    _need_int32("rows", rows)
    tokens, hidden = residual.shape
    if y is not None and (y.dim() != 2 or y.stride(1) != 1 or tuple(y.shape) != (tokens, hidden) or y.dtype != dtype):
        raise KernelShapeError(f"scale_add_norm: y {tuple(y.shape)} {y.dtype} does not fit the stream {(tokens, hidden)} in {dtype}")
    if factor.numel() != hidden or (scale is not None and scale.numel() != hidden):
        raise KernelShapeError(f"scale_add_norm: one factor (and one scale) per column of {hidden}")
    if rows is not None and y is not None:
        raise KernelShapeError("scale_add_norm: rows are picked for the norm alone")
    count = tokens if rows is None else rows.numel()
    cast = torch.empty((count, hidden), dtype=dtype, device=residual.device) if (want_cast or rows is not None) else None
    library.check(
        library.load().mi_scale_add_norm(
            F32 if dtype == torch.float32 else BF16, _ptr(residual), _ptr(y), 0 if y is None else y.stride(0), _ptr(scale),
            _ptr(factor), _ptr(rows), _ptr(cast), count, hidden, float(alpha), float(eps), _stream(),
        )
    )
    return cast


def norm_rows(x: torch.Tensor, weight: torch.Tensor, eps: float, width: int | None = None) -> torch.Tensor:
    """`x[:, :width] * rsqrt(mean(x[:, :width]^2) + eps) * weight` row by row -> [T, width] in the dtype of
    `x` (`weight` float32 [width]; rows of `x` may be wider and strided)."""
    _need_cuda(x, weight)
    _need_contiguous("weight", weight)
    _need_f32("weight", weight)
    width = x.shape[1] if width is None else int(width)
    if x.dim() != 2 or x.stride(1) != 1 or x.shape[1] < width or weight.numel() != width:
        raise KernelShapeError(f"norm_rows: rows of at least {width} columns and as many weights, got {tuple(x.shape)} and {weight.numel()}")
    out = torch.empty((x.shape[0], width), dtype=x.dtype, device=x.device)
    library.check(
        library.load().mi_norm_rows(_dtype_code(x), _ptr(x), x.stride(0), _ptr(weight), _ptr(out), out.stride(0), x.shape[0],
                                    width, float(eps), _stream())
    )
    return out


def qkv_norm_write(
    qkv: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor | None, slot_mapping: torch.Tensor | None,
    k_pages: torch.Tensor | None, v_pages: torch.Tensor | None, *, q_width: int, kv_heads: int, head_dim: int,
    v_head_dim: int, eps: float, v_transposed: bool = False, other_values: torch.Tensor | None = None,
    mix: torch.Tensor | None = None,
) -> None:
    """`qkv` [T, q_width + kv_heads*head_dim + kv_heads*v_head_dim]: q is normed in place over its
    whole width (`q * rsqrt(mean(q^2) + eps) * q_weight`); k, normed the same way with `k_weight`,
    goes to its key-page slot; v goes to its value-page slot, as it is or, with `other_values`
    [T, kv_heads*v_head_dim] (another layer's values of the same tokens) and `mix` (one float32),
    as `(1 - mix) * v + mix * other_values`.  `kv_heads=0`: q only."""
    _need_cuda(qkv, q_weight, k_weight, slot_mapping, k_pages, v_pages, other_values, mix)
    for name, t in (("q_weight", q_weight), ("k_weight", k_weight), ("slot_mapping", slot_mapping),
                    ("k_pages", k_pages), ("v_pages", v_pages)):
        _need_contiguous(name, t)
    _need_int32("slot_mapping", slot_mapping)
    _need_f32("q_weight", q_weight)
    _need_f32("k_weight", k_weight)
    _need_f32("mix", mix)
    if qkv.dim() != 2 or qkv.stride(1) != 1 or qkv.shape[1] < q_width + kv_heads * (head_dim + v_head_dim):
        raise KernelShapeError(f"qkv_norm_write: rows hold q, k and v, got {tuple(qkv.shape)} strides {qkv.stride()}")
    if q_weight.numel() != q_width or (kv_heads > 0 and (k_weight is None or k_weight.numel() != kv_heads * head_dim)):
        raise KernelShapeError("qkv_norm_write: one norm weight per column of q and of k")
    tokens = qkv.shape[0]
    page_size = num_pages = 0
    if kv_heads > 0:
        if slot_mapping is None or k_pages is None or v_pages is None:
            raise KernelShapeError("writing keys and values needs slot_mapping, k_pages and v_pages")
        if k_pages.dtype != qkv.dtype or v_pages.dtype != qkv.dtype:
            raise KernelShapeError(f"pages are {k_pages.dtype}, activations {qkv.dtype}")
        if k_pages.dim() != 4 or k_pages.shape[1] != kv_heads or k_pages.shape[3] != head_dim:
            raise KernelShapeError(f"pages must be [num_pages, {kv_heads}, page_size, {head_dim}], got {tuple(k_pages.shape)}")
        _check_v_pages(k_pages, v_pages, v_transposed, v_head_dim)
        if slot_mapping.numel() != tokens:
            raise KernelShapeError(f"slot_mapping has {slot_mapping.numel()} entries for {tokens} tokens")
        num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
    if other_values is not None:
        if mix is None or mix.numel() != 1:
            raise KernelShapeError("qkv_norm_write: values to mix in come with one float32 weight")
        if (other_values.dim() != 2 or other_values.stride(1) != 1 or other_values.dtype != qkv.dtype
                or tuple(other_values.shape) != (tokens, kv_heads * v_head_dim)):
            raise KernelShapeError(f"qkv_norm_write: the other values must be {qkv.dtype} [{tokens}, {kv_heads * v_head_dim}], got {tuple(other_values.shape)}")
    library.check(
        library.load().mi_qkv_norm_write(
            _dtype_code(qkv), _ptr(qkv), qkv.stride(0), _ptr(q_weight), _ptr(k_weight), _ptr(other_values),
            0 if other_values is None else other_values.stride(0), _ptr(mix) if other_values is not None else None,
            _ptr(slot_mapping) if kv_heads > 0 else None, _ptr(k_pages) if kv_heads > 0 else None,
            _ptr(v_pages) if kv_heads > 0 else None, tokens, q_width, kv_heads, head_dim, v_head_dim, page_size, num_pages,
            int(v_transposed), float(eps), _stream(),
        )
    )


# ----------------------------------------------------------------------------
# routed experts
# ----------------------------------------------------------------------------

ROUTER_MAX_OUTPUTS = 1024


def route_top_k(
    x: torch.Tensor, router: torch.Tensor, correction: torch.Tensor | None, gate_row: torch.Tensor | None, *, top: int,
    route_scale: float,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor | None]:
    """Per row of `x` [T, W]: scores `softmax(router @ x)` over all router outputs (`router` float32
    [outputs, W]), the `top` outputs with the largest `score + correction` (`correction` float32
    [outputs] or None; the lower index wins a tie) -> their indices int32 [T, top] and weights
    `score * route_scale` float32 [T, top] (not renormalized); with `gate_row` (float32 [W]) also
    `logistic(gate_row . x)` float32 [T]."""
    _need_cuda(x, router, correction, gate_row)
    for name, t in (("router", router), ("correction", correction), ("gate_row", gate_row)):
        _need_contiguous(name, t)
        _need_f32(name, t)
    if x.dim() != 2 or x.stride(1) != 1:
        raise KernelShapeError("route_top_k: rows with unit inner stride")
    tokens, width = x.shape
    if router.dim() != 2 or router.shape[1] != width:
        raise KernelShapeError(f"route_top_k: the router is [outputs, {width}], got {tuple(router.shape)}")
    outputs = router.shape[0]
    if not 0 < top <= outputs or outputs > ROUTER_MAX_OUTPUTS:
        raise KernelShapeError(f"route_top_k: {top} of {outputs} outputs (at most {ROUTER_MAX_OUTPUTS})")
    if correction is not None and correction.numel() != outputs:
        raise KernelShapeError(f"route_top_k: one correction per router output, got {correction.numel()} for {outputs}")
    if gate_row is not None and gate_row.numel() != width:
        raise KernelShapeError(f"route_top_k: the gate row has {gate_row.numel()} entries for {width} columns")
    chosen = torch.empty((tokens, top), dtype=torch.int32, device=x.device)
    weights = torch.empty((tokens, top), dtype=torch.float32, device=x.device)
    gates = torch.empty((tokens,), dtype=torch.float32, device=x.device) if gate_row is not None else None
    library.check(
        library.load().mi_route_top_k(
            _dtype_code(x), _ptr(x), x.stride(0), _ptr(router), _ptr(correction), _ptr(gate_row), _ptr(chosen), _ptr(weights),
            _ptr(gates), tokens, width, outputs, int(top), float(route_scale), _stream(),
        )
    )
    return chosen, weights, gates


def _check_experts(x, gate_up, down, chosen, weights, shared, shared_gate):
    _need_cuda(x, gate_up, down, chosen, weights, shared, shared_gate)
    for name, t in (("gate_up", gate_up), ("down", down), ("chosen", chosen), ("weights", weights), ("shared_gate", shared_gate)):
        _need_contiguous(name, t)
    _need_int32("chosen", chosen)
    _need_f32("weights", weights)
    _need_f32("shared_gate", shared_gate)
    if x.dim() != 2 or x.stride(1) != 1:
        raise KernelShapeError("routed experts: rows with unit inner stride")
    tokens, width = x.shape
    if gate_up.dim() != 3 or down.dim() != 3 or gate_up.shape[2] != width or gate_up.shape[1] % 2 or gate_up.dtype != x.dtype or down.dtype != x.dtype:
        raise KernelShapeError(f"routed experts: gate|up is {x.dtype} [experts, 2*ff, {width}], got {gate_up.dtype} {tuple(gate_up.shape)}")
    experts, ff = gate_up.shape[0], gate_up.shape[1] // 2
    if tuple(down.shape) != (experts, width, ff):
        raise KernelShapeError(f"routed experts: down is [{experts}, {width}, {ff}], got {tuple(down.shape)}")
    if chosen.dim() != 2 or chosen.shape[0] != tokens or tuple(weights.shape) != tuple(chosen.shape):
        raise KernelShapeError("routed experts: chosen and weights are [T, top]")
    if shared is not None and (shared.dim() != 2 or shared.stride(1) != 1 or tuple(shared.shape) != (tokens, width) or shared.dtype != x.dtype
                               or shared_gate is None or shared_gate.numel() != tokens):
        raise KernelShapeError("routed experts: a shared expert's rows are [T, W] and come with one gate a row")
    return tokens, width, experts, ff, chosen.shape[1]


def experts_few_rows(
    x: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor,
    shared: torch.Tensor | None = None, shared_gate: torch.Tensor | None = None,
) -> torch.Tensor:
    """`y[t] = sum_k weights[t, k] * expert_{chosen[t, k]}(x[t]) (+ shared_gate[t] * shared[t])` with
    every (row, chosen expert) pair worked on its own, the expert's weights read by index: two
    launches whatever the rows hold, and nothing the host has to know.  An index past the real
    experts is an identity expert (its output is `x[t]`).  `gate_up` [experts, 2*ff, W] (gate rows,
    then up rows), `down` [experts, W, ff]; an expert is `down(silu(gate(x)) * up(x))`."""
    tokens, width, experts, ff, top = _check_experts(x, gate_up, down, chosen, weights, shared, shared_gate)
    act = torch.empty((tokens * top, ff), dtype=x.dtype, device=x.device)
    out = torch.empty((tokens, width), dtype=x.dtype, device=x.device)
    lib = library.load()
    library.check(lib.mi_expert_gate_up(_dtype_code(x), _ptr(x), x.stride(0), _ptr(gate_up), _ptr(chosen), _ptr(act), tokens,
                                        width, ff, experts, top, _stream()))
    library.check(lib.mi_expert_down_combine(
        _dtype_code(x), _ptr(act), _ptr(down), _ptr(chosen), _ptr(weights), _ptr(x), x.stride(0), _ptr(shared),
        0 if shared is None else shared.stride(0), _ptr(shared_gate), _ptr(out), tokens, width, ff, experts, top, _stream()))
    return out


def experts_by_expert_take(x: torch.Tensor, gate_up: torch.Tensor) -> bool:
    """Whether `experts_by_expert` takes these sizes: rows and expert rows read 16 bytes at a time, and
    a few of them fit a block's staging."""
    if x.dim() != 2 or gate_up.dim() != 3 or x.dtype not in (torch.float32, torch.bfloat16):
        return False
    width, ff = x.shape[1], gate_up.shape[1] // 2
    step = 16 // x.element_size()
    lib = library.load()
    code = _dtype_code(x)
    return (width % step == 0 and ff % step == 0 and x.stride(0) % step == 0 and x.data_ptr() % 16 == 0
            and lib.mi_expert_rows_at_once(code, width) > 0 and lib.mi_expert_rows_at_once(code, ff) > 0)


EXPERT_TILES_MIN_ROWS = 48  # rows an expert gets on average from which on the 64 x 64 tiles are taken
GROUPED_ROWS_STEP = 64  # the sorted form's products run over row counts rounded up to a multiple of this


def experts_by_expert(
    x: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor,
    shared: torch.Tensor | None = None, shared_gate: torch.Tensor | None = None, many_rows: bool | None = None,
) -> torch.Tensor:
    """The same sum as `experts_few_rows`, expert by expert without the host knowing anything: one small
    kernel lists the (row, expert) pairs by expert, then every chosen expert's block streams its
    weights once for up to eight of the expert's rows at a time (the rows wait in LDS), and one kernel adds
    a row's results in the order of its choices.  Four launches; an expert that many rows chose is read once
    per sixteen of them, not once per row.  `many_rows` (default: by the average number of rows an expert
    gets): blocks of 64 features that take 64 of an expert's rows a pass, for prompts (bfloat16)."""
    tokens, width, experts, ff, top = _check_experts(x, gate_up, down, chosen, weights, shared, shared_gate)
    if not experts_by_expert_take(x, gate_up):
        raise KernelShapeError(f"experts_by_expert: rows of {width} and {ff} are not read 16 bytes at a time, or do not fit")
    pairs = tokens * top
    listed = torch.empty((pairs,), dtype=torch.int32, device=x.device)
    first = torch.empty((experts + 1,), dtype=torch.int32, device=x.device)
    act = torch.empty((pairs, ff), dtype=x.dtype, device=x.device)
    made = torch.empty((pairs, width), dtype=x.dtype, device=x.device)
    out = torch.empty((tokens, width), dtype=x.dtype, device=x.device)
    lib, code = library.load(), _dtype_code(x)
    if many_rows is None:
        many_rows = pairs >= EXPERT_TILES_MIN_ROWS * experts
    many = int(bool(many_rows))
    library.check(lib.mi_expert_sort(_ptr(chosen), _ptr(listed), _ptr(first), pairs, experts, _stream()))
    library.check(lib.mi_expert_rows(code, 1, _ptr(x), x.stride(0), top, _ptr(gate_up), _ptr(listed), _ptr(first), _ptr(act), ff,
                                     experts, width, ff, many, _stream()))
    library.check(lib.mi_expert_rows(code, 0, _ptr(act), ff, 1, _ptr(down), _ptr(listed), _ptr(first), _ptr(made), width,
                                     experts, ff, width, many, _stream()))
    library.check(lib.mi_expert_combine(
        code, _ptr(made), None, _ptr(chosen), _ptr(weights), _ptr(x), x.stride(0), _ptr(shared),
        0 if shared is None else shared.stride(0), _ptr(shared_gate), _ptr(out), tokens, width, experts, top, _stream()))
    return out


def experts_grouped(
    x: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor,
    shared: torch.Tensor | None = None, shared_gate: torch.Tensor | None = None,
) -> torch.Tensor:
    """The same sum for many rows: the (row, expert) pairs are sorted by expert, every expert that
    was chosen runs its two products once over all its rows (the engine's own products, so each
    expert's weights are read once), and one kernel adds a row's results in the order of its
    choices.  The host reads how many rows each expert got, so this form is not for a step that
    is being recorded."""
    tokens, width, experts, ff, top = _check_experts(x, gate_up, down, chosen, weights, shared, shared_gate)
    flat = chosen.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=experts)[:experts].tolist()
    where = torch.empty_like(order, dtype=torch.int32)
    where[order] = torch.arange(order.numel(), dtype=torch.int32, device=x.device)
    real = sum(counts)
    if x.dtype == torch.bfloat16:
        # The vendor library's product expert by expert, straight into one buffer for all experts' rows, one
        # activation launch.  Every product runs over its expert's rows rounded UP to a multiple of 64: the
        # library looks its kernel up anew for every row count it has not seen (some 50 us of host time, more
        # than the product takes), and experts get a different count every step.  The rows past an expert's
        # last belong to the next expert, whose own product, launched behind this one, writes them again;
        # past the last expert's they are spare rows that nobody reads.
        step = GROUPED_ROWS_STEP
        pairs = order.numel()
        sorted_rows = torch.empty((pairs + step, width), dtype=x.dtype, device=x.device)
        sorted_rows[pairs:].zero_()
        torch.index_select(x, 0, torch.div(order, top, rounding_mode="floor"), out=sorted_rows[:pairs])
        stacked = torch.empty((real + step, 2 * ff), dtype=x.dtype, device=x.device)
        rows = torch.empty((real + step, width), dtype=x.dtype, device=x.device)
        at = 0
        for e, count in enumerate(counts):
            if count:
                upto = at + -(-count // step) * step
                torch.matmul(sorted_rows[at:upto], gate_up[e].t(), out=stacked[at:upto])
                at += count
        stacked[real:].zero_()
        act = silu_mul(stacked)
        at = 0
        for e, count in enumerate(counts):
            if count:
                upto = at + -(-count // step) * step
                torch.matmul(act[at:upto], down[e].t(), out=rows[at:upto])
                at += count
    else:
        sorted_rows = x.index_select(0, torch.div(order, top, rounding_mode="floor"))
        made, at = [], 0
        for e, count in enumerate(counts):
            if count:
                made.append(linear(linear_swiglu(sorted_rows[at:at + count], gate_up[e]), down[e]))
                at += count
        rows = torch.cat(made, dim=0) if made else torch.empty((1, width), dtype=x.dtype, device=x.device)
    out = torch.empty((tokens, width), dtype=x.dtype, device=x.device)
    library.check(library.load().mi_expert_combine(
        _dtype_code(x), _ptr(rows), _ptr(where), _ptr(chosen), _ptr(weights), _ptr(x), x.stride(0), _ptr(shared),
        0 if shared is None else shared.stride(0), _ptr(shared_gate), _ptr(out), tokens, width, experts, top, _stream()))
    return out
