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


def _check_v_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, v_transposed: bool) -> None:
    pages, heads, page_size, head_dim = k_pages.shape
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


def embed_gather(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """`float32(table[ids])`: the start of the residual stream, [T, H] float32."""
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
            _stream(),
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
) -> None:
    """Rotate q in place inside `qkv`; rotate k and write k, v into their page slots.

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
    if qkv.shape[1] < (q_heads + 2 * kv_heads) * head_dim:
        raise KernelShapeError(
            f"qkv rows hold {qkv.shape[1]} values, fewer than (q+2kv)*head_dim = "
            f"{(q_heads + 2 * kv_heads) * head_dim}"
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
        _check_v_pages(k_pages, v_pages, v_transposed)
        if slot_mapping.numel() != tokens:
            raise KernelShapeError(f"slot_mapping has {slot_mapping.numel()} entries for {tokens} tokens")
        num_pages, page_size = k_pages.shape[0], k_pages.shape[2]
    lib = library.load()
    library.check(
        lib.mi_rope_kv_write(
            _dtype_code(qkv), _ptr(qkv), qkv.stride(0), _ptr(cos), _ptr(sin), _ptr(slot_mapping),
            _ptr(k_pages), _ptr(v_pages), tokens, q_heads, kv_heads, head_dim, rotary_dim,
            int(interleaved), page_size, num_pages, int(v_transposed), _stream(),
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
) -> torch.Tensor | AttentionPieces:
    """Causal attention of every token over its request's pages; returns [T, q_heads*head_dim].

    `slopes` (float32 [q_heads], optional): the score of head h for the key at position j
    seen from position p gets `slopes[h] * (j - p)` added before the softmax.  Only the
    plain kernel knows it.

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
        if use_mfma:
            raise KernelShapeError("the matrix-core attention kernel takes no score slopes; keep values untransposed")

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
                int(window or 0), splits, shape, 0, 0, 1, _stream(),
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
                    0 if (leave_pieces and splits > 1) else 1, _stream(),
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
            pieces = run(0, num_requests, leave_pieces=not combine and leading_single == num_requests)
            if pieces is not None:
                return pieces
        return out

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
