"""Each HIP kernel alone against a plain reference, at other sizes than the engine's tiny models."""

import math

import numpy as np
import pytest
import torch

import plain_llama as pl

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype, scale=1.0):
    return (2e-5 if dtype == torch.float32 else 2e-2) * scale


def _rand(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def _off_the_cache_lines(w):
    """A contiguous copy of `w` that begins 16 bytes past a 128-byte boundary.  The weight-streaming
    products read whole cache lines where the rows of the matrix begin on such boundaries (and K
    gives every wave an even number of 32-element steps), half lines otherwise: both ways add
    the same products in the same order, so their results are equal bit for bit."""
    flat = torch.empty(w.numel() + 64, dtype=w.dtype, device=w.device)
    shift = (-(flat.data_ptr() // w.element_size()) % 64 + 8) % 64
    out = flat[shift : shift + w.numel()].view(w.shape)
    assert out.data_ptr() % 128 == 16 and out.is_contiguous()
    out.copy_(w)
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,vocab", [(4096, 1000), (100, 301), (90, 17)])
def test_embed_gather(dtype, hidden, vocab):
    from mini_infer_amd import ops

    table = _rand(vocab, hidden, dtype=dtype)
    ids = torch.tensor([0, vocab - 1, 5, 5, vocab // 2], dtype=torch.int32, device=DEV)
    out = ops.embed_gather(table, ids)
    assert out.dtype == torch.float32
    assert torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [4096, 100, 90, 9000, 1000])
@pytest.mark.parametrize("tokens", [7, 300])  # few rows; the rows of a prompt's portion
def test_add_rmsnorm(dtype, hidden, tokens):
    from mini_infer_amd import ops

    eps = 3e-6
    residual = _rand(tokens, hidden, seed=1, scale=2.0)
    delta = _rand(tokens, hidden, dtype=dtype, seed=2)
    weight = (_rand(hidden, seed=3) * 0.2 + 1.0).to(dtype)
    expected_sum = residual.double() + delta.double()
    expected = pl.rms_norm(expected_sum.cpu().numpy(), weight.double().cpu().numpy(), eps)

    res = residual.clone()
    out = ops.add_rmsnorm(delta, res, weight, eps)
    assert torch.allclose(res, expected_sum.float(), atol=1e-6)  # the sum is stored, in float32
    assert np.abs(out.float().cpu().numpy() - expected).max() < _tol(dtype, 4)

    # first layer: nothing to add, residual untouched
    res = residual.clone()
    out = ops.add_rmsnorm(None, res, weight, eps)
    assert torch.equal(res, residual)
    plain = pl.rms_norm(residual.double().cpu().numpy(), weight.double().cpu().numpy(), eps)
    assert np.abs(out.float().cpu().numpy() - plain).max() < _tol(dtype, 4)

    # chosen rows only: the residual stays as it was
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    res = residual.clone()
    out = ops.add_rmsnorm(delta, res, weight, eps, rows)
    assert torch.equal(res, residual) and out.shape == (3, hidden)
    assert np.abs(out.float().cpu().numpy() - expected[[5, 0, 5]]).max() < _tol(dtype, 4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter", [14336, 130, 7, 136])
@pytest.mark.parametrize("tokens", [5, 300])  # few rows; the rows of a prompt's portion
def test_silu_mul(dtype, inter, tokens):
    from mini_infer_amd import ops

    gate_up = _rand(tokens, 2 * inter, dtype=dtype, seed=4, scale=3.0)
    gate_up[0, 0] = 0.0
    gate_up[0, 1 % inter] = 80.0
    gate_up[1, 0] = -80.0
    out = ops.silu_mul(gate_up).float().cpu().numpy()
    g = gate_up[:, :inter].double().cpu().numpy()
    u = gate_up[:, inter:].double().cpu().numpy()
    expected = pl.silu(g) * u
    assert np.isfinite(out).all()
    assert np.abs(out - expected).max() < _tol(dtype, max(1.0, np.abs(expected).max()))
    assert out[0, 0] == 0.0


@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (7, 130, 90), (65, 301, 259), (300, 96, 4096), (33, 1, 5)])
def test_gemm_f32_is_true_float32(m, n, k):
    from mini_infer_amd import ops

    a, w = _rand(m, k, seed=5), _rand(n, k, seed=6)
    out = ops.gemm_f32(a, w)
    expected = a.double() @ w.double().T
    # float32 rounding of a K-long sum; a reduced-precision matrix mode (10-bit or
    # 7-bit mantissas) would miss this bound by a factor of ten or more
    assert (out.double() - expected).abs().max() < 6e-8 * math.sqrt(k) * float(expected.abs().max()) * 4
    # a row's result does not depend on the other rows in the batch
    alone = ops.gemm_f32(a[m // 2 : m // 2 + 1].contiguous(), w)
    assert torch.equal(alone[0], out[m // 2])
    # strided rows
    wide = _rand(m, k + 3, seed=7)
    assert torch.equal(ops.gemm_f32(wide[:, :k], w), ops.gemm_f32(wide[:, :k].contiguous(), w))


@pytest.mark.parametrize(
    "m,n,k",
    [(1, 4096, 4096), (8, 6144, 4096), (16, 96, 64), (7, 301, 96), (13, 130, 160), (16, 1000, 14336),
     (5, 128256, 256), (3, 7, 32), (9, 28672, 4096), (2, 16400, 1056), (4, 4096, 1536), (6, 640, 3072), (16, 2050, 512)],
)
def test_gemm_skinny_bf16(m, n, k):
    from mini_infer_amd import ops

    a, w = _rand(m, k, dtype=torch.bfloat16, seed=9), _rand(n, k, dtype=torch.bfloat16, seed=10, scale=0.05)
    out = ops.gemm_skinny_bf16(a, w)
    expected = a.double() @ w.double().T
    # float32 accumulation of exact bfloat16 products, one rounding to bfloat16 at the end
    assert (out.double() - expected).abs().max() < 2.0 ** -8 * float(expected.abs().max()) + 1e-6
    # a row's result does not depend on the other rows in the batch
    alone = ops.gemm_skinny_bf16(a[m // 2 : m // 2 + 1].contiguous(), w)
    assert torch.equal(alone[0], out[m // 2])
    # strided activations (a slice of a wider buffer), and the dispatch in `linear`
    wide = _rand(m, k + 8, dtype=torch.bfloat16, seed=11)
    assert torch.equal(ops.gemm_skinny_bf16(wide[:, :k], w), ops.gemm_skinny_bf16(wide[:, :k].contiguous(), w))
    assert torch.equal(ops.linear(a, w), out)
    assert torch.equal(ops.gemm_skinny_bf16(a, _off_the_cache_lines(w)), out)


@pytest.mark.parametrize(
    "m,n,k",
    [(1, 4096, 14336), (8, 1000, 8192 + 32), (16, 4096, 4096), (17, 1003, 4096), (33, 136, 608), (64, 4096, 14336),
     (47, 5, 32), (64, 260, 8192 - 224), (128, 4096, 4096), (101, 200, 1024 + 64), (24, 3072, 8192 + 64)],
)
def test_linear_in_partial_sums_then_norm_is_linear_then_norm(m, n, k):
    """A product left as sums over ranges of K, added up by the norm that follows it: the
    same residual and output, bit for bit, as with the pieces added first (`finish`), and the
    product itself within float32 accumulation of the exact one; a row's pieces do not
    depend on the other rows."""
    from mini_infer_amd import ops

    a, w = _rand(m, k, dtype=torch.bfloat16, seed=31), _rand(n, k, dtype=torch.bfloat16, seed=32, scale=0.05)
    partial = ops.linear_partial_sums(a, w)
    assert partial.pieces.dtype == torch.float32 and partial.pieces.shape[1:] == (m, n)
    delta = partial.finish()
    expected = a.double() @ w.double().T
    assert (delta.double() - expected).abs().max() < 2.0 ** -8 * float(expected.abs().max()) + 1e-6
    alone = ops.linear_partial_sums(a[m // 2 : m // 2 + 1].contiguous(), w)
    assert torch.equal(alone.pieces[:, 0], partial.pieces[:, m // 2])
    # strided activations: a slice of a wider buffer
    wide = _rand(m, k + 8, dtype=torch.bfloat16, seed=35)
    assert torch.equal(ops.linear_partial_sums(wide[:, :k], w).pieces, ops.linear_partial_sums(wide[:, :k].contiguous(), w).pieces)
    assert torch.equal(ops.linear_partial_sums(a, _off_the_cache_lines(w)).pieces, partial.pieces)
    weight = _rand(n, dtype=torch.bfloat16, seed=33).abs() + 0.5
    for rows in (None, torch.tensor([m - 1, 0], dtype=torch.int32, device=DEV)):
        res_a, res_b = _rand(m, n, seed=34), _rand(m, n, seed=34)
        out_a = ops.add_rmsnorm(partial, res_a, weight, 1e-5, rows)
        out_b = ops.add_rmsnorm(delta, res_b, weight, 1e-5, rows)
        assert torch.equal(out_a, out_b) and torch.equal(res_a, res_b)


def test_linear_leaves_partial_sums_only_where_asked_and_where_it_pays():
    from mini_infer_amd import ops
    from mini_infer_amd.exceptions import KernelShapeError

    a, w = _rand(12, 12288, dtype=torch.bfloat16, seed=36), _rand(64, 12288, dtype=torch.bfloat16, seed=37, scale=0.05)
    assert ops.partial_sums_pay(12, 64, 12288) and isinstance(ops.linear(a, w, partial_ok=True), ops.PartialSums)
    assert isinstance(ops.linear(a, w), torch.Tensor)
    assert not ops.partial_sums_pay(8, 64, 12288) and not ops.partial_sums_pay(12, 8192, 12288) and ops.partial_sums_pay(15, 8192, 12288)
    assert not ops.partial_sums_pay(16, 64, 4096) and ops.partial_sums_pay(17, 64, 4096)
    assert not ops.partial_sums_pay(4, 64, 12288) and not ops.partial_sums_pay(16, 3072, 8192)
    assert not ops.partial_sums_pay(129, 64, 12288) and not ops.partial_sums_pay(8, 28672, 12288)
    assert isinstance(ops.linear(a[:, :4096].contiguous(), w[:, :4096].contiguous(), partial_ok=True), torch.Tensor)
    assert isinstance(ops.linear(a.float(), w.float(), partial_ok=True), torch.Tensor)
    partial = ops.linear(a, w, partial_ok=True)
    with pytest.raises(KernelShapeError, match="partial sums"):
        ops.add_rmsnorm(ops.PartialSums(partial.pieces[:, :1].contiguous(), torch.bfloat16), _rand(8, 64),
                        _rand(64, dtype=torch.bfloat16), 1e-5)
    with pytest.raises(KernelShapeError, match="1 to 128 rows"):
        ops.linear_partial_sums(_rand(129, 64, dtype=torch.bfloat16), _rand(16, 64, dtype=torch.bfloat16))


@pytest.mark.parametrize(
    "m,inter,k",
    [(1, 14336, 4096), (8, 14336, 4096), (16, 160, 64), (7, 301, 96), (13, 4100, 160), (3, 5, 32), (9, 8192, 3072),
     (5, 520, 1536), (2, 24, 512), (17, 14336, 4096), (32, 8192, 3072), (24, 160, 64), (31, 301, 96), (20, 520, 1536)],
)
def test_linear_swiglu_is_the_product_followed_by_the_activation(m, inter, k):
    from mini_infer_amd import ops

    a = _rand(m, k, dtype=torch.bfloat16, seed=12)
    w = _rand(2 * inter, k, dtype=torch.bfloat16, seed=13, scale=0.08)
    fused = ops.linear_swiglu(a, w)
    assert fused.shape == (m, inter)
    # the two-kernel path: the product (rounded to bfloat16), then the activation (the plain
    # weight-streaming product takes 16 rows; a row's result does not depend on the others)
    for first in range(0, m, 16):
        assert torch.equal(fused[first : first + 16], ops.silu_mul(ops.gemm_skinny_bf16(a[first : first + 16], w)))
    assert torch.equal(ops.linear_swiglu(a, _off_the_cache_lines(w)), fused)
    gate_up = (a.double() @ w.double().T).bfloat16().double()
    gate, up = gate_up[:, :inter], gate_up[:, inter:]
    expected = gate / (1 + torch.exp(-gate)) * up
    assert (fused.double() - expected).abs().max() < 2.0 ** -7 * float(expected.abs().max()) + 1e-6
    # more rows than the fused kernel takes: the same function, through the library product
    many = _rand(40, k, dtype=torch.bfloat16, seed=14)
    assert ops.linear_swiglu(many, w).shape == (40, inter)
    # float32 goes through the true float32 product
    got32 = ops.linear_swiglu(a.float(), w.float())
    exact = a.double() @ w.double().T
    exact = exact[:, :inter] / (1 + torch.exp(-exact[:, :inter])) * exact[:, inter:]
    assert (got32.double() - exact).abs().max() < 1e-4 * float(exact.abs().max()) + 1e-6


@pytest.mark.parametrize("v_transposed", [False, True])
@pytest.mark.parametrize(
    "m,hidden,q_heads,kv_heads,head_dim,page_size",
    [(8, 4096, 32, 8, 128, 16), (1, 4096, 32, 8, 128, 16), (16, 96, 3, 1, 32, 16), (5, 160, 6, 2, 64, 32), (9, 64, 4, 4, 96, 48),
     (3, 1536, 6, 2, 64, 16), (17, 4096, 32, 8, 128, 16), (32, 1536, 6, 2, 64, 16), (25, 96, 3, 1, 32, 16)],
)
def test_qkv_rope_write_is_the_product_followed_by_rotation_and_cache_write(
    v_transposed, m, hidden, q_heads, kv_heads, head_dim, page_size
):
    from mini_infer_amd import ops

    num_pages = 7
    width = (q_heads + 2 * kv_heads) * head_dim
    x = _rand(m, hidden, dtype=torch.bfloat16, seed=31)
    w = _rand(width, hidden, dtype=torch.bfloat16, seed=32, scale=0.1)
    positions = torch.tensor(([0, 1, 700, 5, 131071, 17, 18, 19, 3000, 2, 4, 6, 8, 10, 12, 14] + list(range(50, 66)))[:m],
                             dtype=torch.int32, device=DEV)
    inv_freq = torch.from_numpy(pl.inv_freq_default(head_dim, 500000.0)).to(DEV)
    cos, sin = ops.rope_table(positions, inv_freq)
    slots = torch.tensor(([40, 3, 17, 16, 0, 43, -1, 9, 22, 5, 6, 7, 30, 31, 32, 33] + list(range(60, 76)))[:m],
                         dtype=torch.int32, device=DEV)
    slots = torch.where(slots >= 0, slots % (num_pages * page_size), slots)
    assert len(set(slots[slots >= 0].tolist())) == int((slots >= 0).sum())  # (no two rows write one slot)

    def pages():
        k = torch.full((num_pages, kv_heads, page_size, head_dim), 7.0, dtype=torch.bfloat16, device=DEV)
        v_shape = (num_pages, kv_heads, head_dim, page_size) if v_transposed else k.shape
        return k, torch.full(v_shape, 7.0, dtype=torch.bfloat16, device=DEV)

    k_two, v_two = pages()
    qkv = torch.cat([ops.gemm_skinny_bf16(x[first : first + 16], w) for first in range(0, m, 16)])
    ops.rope_kv_write(qkv, cos, sin, slots, k_two, v_two, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
                      rotary_dim=head_dim, interleaved=False, v_transposed=v_transposed)
    k_one, v_one = pages()
    queries = ops.qkv_rope_write(x, w, cos, sin, slots, k_one, v_one, q_heads=q_heads, kv_heads=kv_heads,
                                 head_dim=head_dim, v_transposed=v_transposed)
    assert queries.shape == (m, q_heads * head_dim)
    # the same products rounded the same way, the same rotation formula: equal up to how the
    # compiler contracts a multiply-add before the final rounding
    tol = 2.0 ** -7 * float(qkv.float().abs().max())
    assert (queries.float() - qkv[:, : q_heads * head_dim].float()).abs().max() <= tol
    assert (k_one.float() - k_two.float()).abs().max() <= tol
    assert torch.equal(v_one, v_two)  # values are copied, not rotated
    k_off, v_off = pages()
    off_lines = ops.qkv_rope_write(x, _off_the_cache_lines(w), cos, sin, slots, k_off, v_off, q_heads=q_heads,
                                   kv_heads=kv_heads, head_dim=head_dim, v_transposed=v_transposed)
    assert torch.equal(off_lines, queries) and torch.equal(k_off, k_one) and torch.equal(v_off, v_one)
    # queries only (a layer that reads another layer's keys and values): pages stay untouched
    k_none, v_none = pages()
    only_q = ops.qkv_rope_write(x, w[: q_heads * head_dim], cos, sin, None, k_none, v_none, q_heads=q_heads,
                                kv_heads=0, head_dim=head_dim, v_transposed=v_transposed)
    assert torch.equal(only_q, queries)
    assert torch.all(k_none == 7.0) and torch.all(v_none == 7.0)


def test_linear_falls_back_to_the_library_where_the_skinny_kernel_does_not_apply():
    from mini_infer_amd import ops
    from mini_infer_amd.exceptions import KernelShapeError

    a, w = _rand(5, 90, dtype=torch.bfloat16), _rand(40, 90, dtype=torch.bfloat16, seed=1)
    assert (ops.linear(a, w).double() - a.double() @ w.double().T).abs().max() < 0.2
    big = _rand(100, 64, dtype=torch.bfloat16)
    assert ops.linear(big, _rand(32, 64, dtype=torch.bfloat16, seed=2)).shape == (100, 32)
    with pytest.raises(KernelShapeError, match="m <= 16"):
        ops.gemm_skinny_bf16(big, _rand(32, 64, dtype=torch.bfloat16, seed=2))
    with pytest.raises(KernelShapeError):
        ops.gemm_skinny_bf16(a, w)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(
    "q_heads,kv_heads,head_dim,rotary_dim,interleaved",
    [(32, 8, 128, 128, False), (3, 1, 32, 32, False), (6, 3, 48, 16, False), (4, 2, 64, 64, True), (2, 2, 16, 0, False),
     (5, 1, 40, 24, False)],
)
@pytest.mark.parametrize("tokens", [9, 300])  # few rows; the rows of a prompt's portion
def test_rope_kv_write(dtype, q_heads, kv_heads, head_dim, rotary_dim, interleaved, tokens):
    from mini_infer_amd import ops

    page_size = 4
    num_pages = tokens + 2
    width = (q_heads + 2 * kv_heads) * head_dim
    qkv = _rand(tokens, width, dtype=dtype, seed=8)
    original = qkv.clone()
    rng = np.random.default_rng(tokens)
    some = [0, 1, 2, 3, 700, 701, 5, 6, 131071]
    positions = torch.tensor(some + rng.integers(0, 131072, tokens - len(some)).tolist(), dtype=torch.int32, device=DEV)
    half = rotary_dim // 2
    if half:
        inv_freq = torch.from_numpy(pl.inv_freq_default(rotary_dim, 500000.0)).to(DEV)
        cos, sin = ops.rope_table(positions, inv_freq)
        angle = positions.float().cpu().numpy()[:, None] * inv_freq.cpu().numpy()[None, :]
        assert np.abs(cos.cpu().numpy() - np.cos(angle.astype(np.float64))).max() < 2e-6
        assert np.abs(sin.cpu().numpy() - np.sin(angle.astype(np.float64))).max() < 2e-6
    else:
        cos = sin = torch.empty((tokens, 0), dtype=torch.float32, device=DEV)
    # scattered slots, one token not written at all
    more = [int(x) for x in rng.permutation(num_pages * page_size) if x not in (40, 3, 17, 16, 0, 43, 9, 22)]
    slots = torch.tensor([40, 3, 17, 16, 0, 43, -1, 9, 22] + more[: tokens - 9], dtype=torch.int32, device=DEV)
    k_pages = torch.zeros((num_pages, kv_heads, page_size, head_dim), dtype=dtype, device=DEV)
    v_pages = torch.zeros_like(k_pages)
    ops.rope_kv_write(qkv, cos, sin, slots, k_pages, v_pages, q_heads=q_heads, kv_heads=kv_heads,
                      head_dim=head_dim, rotary_dim=rotary_dim, interleaved=interleaved)
    # the same write with values transposed inside each page
    vt_pages = torch.zeros((num_pages, kv_heads, head_dim, page_size), dtype=dtype, device=DEV)
    ops.rope_kv_write(original.clone(), cos, sin, slots, torch.zeros_like(k_pages), vt_pages, q_heads=q_heads,
                      kv_heads=kv_heads, head_dim=head_dim, rotary_dim=rotary_dim, interleaved=interleaved,
                      v_transposed=True)
    assert torch.equal(vt_pages.transpose(2, 3), v_pages)

    def rotate(x):  # x [T, heads, D] float64
        if not half:
            return x
        c, s = cos.double().cpu().numpy()[:, None, :], sin.double().cpu().numpy()[:, None, :]
        out = x.copy()
        if interleaved:
            x0, x1 = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
            out[..., 0:rotary_dim:2], out[..., 1:rotary_dim:2] = x0 * c - x1 * s, x1 * c + x0 * s
        else:
            x0, x1 = x[..., :half], x[..., half:rotary_dim]
            out[..., :half], out[..., half:rotary_dim] = x0 * c - x1 * s, x1 * c + x0 * s
        return out

    src = original.double().cpu().numpy()
    q_in = src[:, : q_heads * head_dim].reshape(tokens, q_heads, head_dim)
    k_in = src[:, q_heads * head_dim : (q_heads + kv_heads) * head_dim].reshape(tokens, kv_heads, head_dim)
    v_in = src[:, (q_heads + kv_heads) * head_dim :].reshape(tokens, kv_heads, head_dim)
    got_q = qkv[:, : q_heads * head_dim].double().cpu().numpy().reshape(tokens, q_heads, head_dim)
    assert np.abs(got_q - rotate(q_in)).max() < _tol(dtype, 4)
    assert torch.equal(qkv[:, q_heads * head_dim :], original[:, q_heads * head_dim :])  # k, v inputs untouched
    expect_k = np.zeros(k_pages.shape)
    expect_v = np.zeros(v_pages.shape)
    rk = rotate(k_in)
    for t, slot in enumerate(slots.tolist()):
        if slot >= 0:
            expect_k[slot // page_size, :, slot % page_size] = rk[t]
            expect_v[slot // page_size, :, slot % page_size] = v_in[t]
    assert np.abs(k_pages.double().cpu().numpy() - expect_k).max() < _tol(dtype, 4)
    assert np.array_equal(v_pages.double().cpu().numpy(), expect_v)  # values copied bit for bit, other slots still zero
    if half:
        # position 0 leaves q as it was
        assert torch.equal(qkv[0, : q_heads * head_dim], original[0, : q_heads * head_dim])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [16, 8])
@pytest.mark.parametrize("more_pages", [0, 40])  # 40 more whole pages: the rows of a prompt's portion
def test_rope_kv_write_whole_pages_of_transposed_values(dtype, page_size, more_pages):
    """Tokens that fill a page in order have their transposed values written a whole page at a
    time by the page's first token; pages filled out of order, from the middle, or only in
    part go token by token.  All give what the plain layout gives, transposed."""
    from mini_infer_amd import ops

    q_heads, kv_heads, head_dim, num_pages = 4, 2, 32, 7 + more_pages
    ps = page_size
    slots = (
        list(range(2 * ps, 3 * ps))  # page 2, in order: written at once
        + [0 * ps + i for i in np.random.default_rng(0).permutation(ps)]  # page 0, out of order
        + list(range(4 * ps + 3, 4 * ps + 3 + 5))  # page 4 from its middle
        + list(range(5 * ps, 5 * ps + ps // 2))  # half of page 5
        + [-1]  # a token that is not written
        + list(range(6 * ps, 7 * ps))  # page 6, in order, at the very end of the step
        + list(range(3 * ps, 3 * ps + ps - 1))  # page 3 but for its last slot
        + list(range(7 * ps, (7 + more_pages) * ps))  # (a token too late to start on a page's edge)
    )
    tokens = len(slots)
    qkv = _rand(tokens, (q_heads + 2 * kv_heads) * head_dim, dtype=dtype, seed=21)
    positions = torch.arange(tokens, dtype=torch.int32, device=DEV)
    cos, sin = ops.rope_table(positions, torch.from_numpy(pl.inv_freq_default(head_dim, 10000.0)).to(DEV))
    slot_t = torch.tensor(slots, dtype=torch.int32, device=DEV)
    k_a = torch.zeros((num_pages, kv_heads, ps, head_dim), dtype=dtype, device=DEV)
    v_a = torch.zeros_like(k_a)
    ops.rope_kv_write(qkv.clone(), cos, sin, slot_t, k_a, v_a, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
                      rotary_dim=head_dim, interleaved=False)
    k_b = torch.zeros_like(k_a)
    v_b = torch.zeros((num_pages, kv_heads, head_dim, ps), dtype=dtype, device=DEV)
    ops.rope_kv_write(qkv.clone(), cos, sin, slot_t, k_b, v_b, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
                      rotary_dim=head_dim, interleaved=False, v_transposed=True)
    assert torch.equal(k_a, k_b) and torch.equal(v_b.transpose(2, 3), v_a)
    values = qkv[:, (q_heads + kv_heads) * head_dim :].reshape(tokens, kv_heads, head_dim)
    for t, slot in enumerate(slots):
        if slot >= 0:
            assert torch.equal(v_a[slot // ps, :, slot % ps], values[t])
    assert int((v_a != 0).any(dim=-1).sum()) == sum(1 for s in slots if s >= 0) * kv_heads  # nothing else was written


def _paged_case(dtype, q_heads, kv_heads, head_dim, page_size, lengths, q_lens, seed=0, v_transposed=False):
    """Random keys/values scattered over shuffled pages; queries are the last q_len positions."""
    rng = np.random.default_rng(seed)
    num_requests = len(lengths)
    pages_per = [-(-n // page_size) for n in lengths]
    num_pages = sum(pages_per) + 3
    order = rng.permutation(num_pages)
    max_blocks = max(pages_per)
    table = np.full((num_requests, max_blocks), -1, dtype=np.int32)
    k_pages = torch.zeros((num_pages, kv_heads, page_size, head_dim), dtype=dtype)
    v_pages = torch.zeros_like(k_pages)
    ks, vs, qs, token_request, positions = [], [], [], [], []
    at = 0
    for b, n in enumerate(lengths):
        table[b, : pages_per[b]] = order[at : at + pages_per[b]]
        at += pages_per[b]
        k = torch.from_numpy(rng.standard_normal((n, kv_heads, head_dim))).to(dtype)
        v = torch.from_numpy(rng.standard_normal((n, kv_heads, head_dim))).to(dtype)
        at_page = torch.from_numpy(table[b, np.arange(n) // page_size].astype(np.int64))
        at_slot = torch.arange(n) % page_size
        k_pages[at_page, :, at_slot] = k
        v_pages[at_page, :, at_slot] = v
        q = torch.from_numpy(rng.standard_normal((q_lens[b], q_heads, head_dim))).to(dtype)
        ks.append(k), vs.append(v), qs.append(q)
        token_request += [b] * q_lens[b]
        positions += list(range(n - q_lens[b], n))
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    if v_transposed:
        v_pages = v_pages.transpose(2, 3).contiguous()
    return dict(
        q=torch.cat(qs).reshape(-1, q_heads * head_dim).to(DEV), qs=qs, ks=ks, vs=vs,
        k_pages=k_pages.to(DEV), v_pages=v_pages.to(DEV), v_transposed=v_transposed,
        cu=torch.tensor(cu, dtype=torch.int32, device=DEV), host_cu=cu,
        block_table=torch.from_numpy(table).to(DEV),
        token_request=torch.tensor(token_request, dtype=torch.int32, device=DEV),
        positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
    )


def _attend(case, q_heads, kv_heads, head_dim, scale, window, max_seq_len):
    from mini_infer_amd import ops

    return ops.paged_attention(
        case["q"], case["k_pages"], case["v_pages"], case["block_table"], case["token_request"],
        case["positions"], case["cu"], case["host_cu"], q_heads=q_heads, kv_heads=kv_heads,
        head_dim=head_dim, scale=scale, window=window, max_seq_len=max_seq_len,
        v_transposed=case["v_transposed"])


def _attention_expected(case, scale, window):
    outs = []
    for q, k, v in zip(case["qs"], case["ks"], case["vs"]):
        out = pl.causal_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), scale, window)
        outs.append(out.reshape(out.shape[0], -1))
    return np.concatenate(outs)


ATTENTION_MODES = [("plain", torch.float32), ("plain", torch.bfloat16), ("mfma", torch.bfloat16)]
PLAIN_SHAPES = [
    (32, 8, 128, 16, None),
    (5, 5, 64, 1, None),
    (7, 1, 16, 4, None),
    (6, 2, 48, 8, 9),
    (10, 2, 80, 64, None),
    (4, 4, 256, 16, 40),
    (12, 2, 112, 32, None),
    # head sizes no 16-byte load divides: read in pairs of elements, every row's end guarded
    (8, 2, 100, 16, None),
    (6, 3, 40, 4, 21),
    (3, 1, 2, 4, None),
    (4, 2, 130, 16, None),
    (5, 1, 254, 8, 50),
]
MFMA_SHAPES = [
    (32, 8, 128, 16, None),
    (3, 1, 32, 16, None),
    (7, 1, 64, 32, None),
    (6, 2, 96, 16, 9),
    (40, 2, 64, 16, None),
    (8, 2, 256, 64, 40),
    (12, 4, 192, 16, None),
    (5, 5, 128, 48, 70),
]


def _attention_cases():
    for mode, dtype in ATTENTION_MODES:
        for shape in MFMA_SHAPES if mode == "mfma" else PLAIN_SHAPES:
            yield pytest.param(mode, dtype, *shape, id=f"{mode}-{str(dtype)[6:]}-" + "-".join(map(str, shape)))


@pytest.mark.parametrize("mode,dtype,q_heads,kv_heads,head_dim,page_size,window", list(_attention_cases()))
def test_paged_attention_mixed_batch(mode, dtype, q_heads, kv_heads, head_dim, page_size, window):
    """Portions of prompts beside single tokens, pages in shuffled order, groups of 1 to 20 heads."""
    lengths, q_lens = [70, 1, 33, 129, 64, 200], [70, 1, 5, 1, 2, 37]
    case = _paged_case(dtype, q_heads, kv_heads, head_dim, page_size, lengths, q_lens, seed=head_dim,
                       v_transposed=mode == "mfma")
    scale = 1.0 / math.sqrt(head_dim)
    out = _attend(case, q_heads, kv_heads, head_dim, scale, window, max(lengths))
    expected = _attention_expected(case, scale, window)
    assert np.abs(out.double().cpu().numpy() - expected).max() < _tol(dtype, 2)


@pytest.mark.parametrize("mode,dtype", ATTENTION_MODES)
@pytest.mark.parametrize("q_heads,kv_heads,window", [(8, 2, None), (40, 2, None), (4, 4, 1000)])
def test_paged_attention_decode_only_splits_keys(mode, dtype, q_heads, kv_heads, window):
    """Single tokens over long contexts: the key range is split over blocks and recombined."""
    from mini_infer_amd import ops

    head_dim, page_size = 128, 16
    lengths, q_lens = [3000, 517, 1, 64, 2049], [1, 1, 1, 1, 1]
    assert ops.attention_splits(5 * kv_heads, max(lengths)) > 1
    case = _paged_case(dtype, q_heads, kv_heads, head_dim, page_size, lengths, q_lens, seed=1,
                       v_transposed=mode == "mfma")
    scale = 0.2
    out = _attend(case, q_heads, kv_heads, head_dim, scale, window, max(lengths))
    expected = _attention_expected(case, scale, window)
    assert np.abs(out.double().cpu().numpy() - expected).max() < _tol(dtype, 2)


@pytest.mark.parametrize("mode,dtype", ATTENTION_MODES)
def test_paged_attention_portion_over_long_context_splits_keys(mode, dtype):
    """A short portion late in a long prompt: few tiles, so keys are split there too."""
    q_heads, kv_heads, head_dim, page_size = 8, 2, 64, 16
    lengths, q_lens = [2500, 900], [40, 3]
    case = _paged_case(dtype, q_heads, kv_heads, head_dim, page_size, lengths, q_lens, seed=2,
                       v_transposed=mode == "mfma")
    out = _attend(case, q_heads, kv_heads, head_dim, 0.15, None, max(lengths))
    expected = _attention_expected(case, 0.15, None)
    assert np.abs(out.double().cpu().numpy() - expected).max() < _tol(dtype, 2)


@pytest.mark.parametrize("mode,dtype", ATTENTION_MODES)
def test_paged_attention_single_tokens_first_then_portions(mode, dtype):
    """The order a scheduler produces: decoding requests (one token each, long and short
    contexts) first, portions of prompts after them.  The matrix-core path runs the two
    runs of requests as two launches over the same buffers."""
    q_heads, kv_heads, head_dim, page_size = 8, 2, 64, 16
    lengths, q_lens = [1500, 17, 640, 300, 90, 33], [1, 1, 1, 140, 90, 2]
    case = _paged_case(dtype, q_heads, kv_heads, head_dim, page_size, lengths, q_lens, seed=4,
                       v_transposed=mode == "mfma")
    out = _attend(case, q_heads, kv_heads, head_dim, 0.15, None, max(lengths))
    expected = _attention_expected(case, 0.15, None)
    assert np.abs(out.double().cpu().numpy() - expected).max() < _tol(dtype, 2)


def test_float32_attention_over_thousands_of_keys_is_rounded_once():
    """The 32-bit path's attention keeps its sums in 64-bit: the output of a row over 2,500 keys
    differs from the exact one by about one float32 rounding (relative 2.5e-8 on average).  A
    float32 sum that is rounded at every key is 6e-7 away at this length, which 32 layers
    turn into logits off by more than 1e-4."""
    q_heads, kv_heads, head_dim, page_size = 8, 2, 128, 16
    lengths, q_lens = [2500, 1800], [300, 1]
    case = _paged_case(torch.float32, q_heads, kv_heads, head_dim, page_size, lengths, q_lens, seed=9)
    scale = 0.35  # scores of a few units either way: some keys stand out, hundreds still count
    out = _attend(case, q_heads, kv_heads, head_dim, scale, None, max(lengths)).double().cpu().numpy()
    expected = _attention_expected(case, scale, None)
    relative = np.linalg.norm(out - expected) / np.linalg.norm(expected)
    assert relative < 6e-8, f"relative error {relative:.2e}"


@pytest.mark.parametrize("m,n,k", [(1, 1000, 256), (8, 333, 96), (16, 4100, 512)])
def test_product_with_float32_output_keeps_its_sums(m, n, k):
    """The output head's product for few bfloat16 rows writes float32 itself: the values of
    `gemm_skinny_bf16`, widened (what the many-row path gives too)."""
    from mini_infer_amd import ops

    a, w = _rand(m, k, dtype=torch.bfloat16, seed=1).to(DEV), _rand(n, k, dtype=torch.bfloat16, seed=2).to(DEV)
    got = ops.linear_f32_out(a, w)
    assert got.dtype == torch.float32 and got.shape == (m, n)
    exact = a.double() @ w.double().T
    assert float((got.double() - exact).abs().max()) < _tol(torch.bfloat16) * k ** 0.5
    assert torch.equal(got, ops.gemm_skinny_bf16(a, w).float())
    # float32 operands and many rows go their own ways to the same kind of result
    assert ops.linear_f32_out(a.float(), w.float()).dtype == torch.float32
    many = _rand(40, k, dtype=torch.bfloat16, seed=3).to(DEV)
    assert ops.linear_f32_out(many, w).dtype == torch.float32


def test_float32_product_is_rounded_once():
    """`gemm_f32` carries its sums in 64-bit: a sum over 14,336 terms is one float32 rounding
    away from exact (2.5e-8 on average), in the many-row and in the few-row kernel alike."""
    from mini_infer_amd import ops

    a = _rand(40, 14336, seed=1).to(DEV)
    w = _rand(96, 14336, seed=2).to(DEV)
    exact = a.double() @ w.double().T
    for rows in (40, 7):
        got = ops.gemm_f32(a[:rows], w).double()
        relative = float((got - exact[:rows]).norm() / exact[:rows].norm())
        assert relative < 4e-8, f"{rows} rows: relative error {relative:.2e}"
    assert torch.equal(ops.gemm_f32(a[:7], w), ops.gemm_f32(a, w)[:7])  # a row's bits do not depend on its company


@pytest.mark.parametrize("mode,dtype", ATTENTION_MODES)
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,window", [(8, 2, 64, None), (32, 8, 128, 50), (6, 3, 96, None)])
def test_paged_attention_with_request_boundaries_known_on_the_device_only(mode, dtype, q_heads, kv_heads, head_dim, window):
    """What a recorded step with portions in it asks of the attention: `host_cu_seqlens_q=None`,
    the launch shaped by the number of tokens and requests alone; requests that bring no token
    (here two, at the end, as the padding of a bucket leaves them) are passed over."""
    from mini_infer_amd import ops

    page_size = 16
    lengths, q_lens = [300, 41, 1500, 90, 64], [70, 1, 1, 33, 2]
    case = _paged_case(dtype, q_heads, kv_heads, head_dim, page_size, lengths, q_lens, seed=21, v_transposed=mode == "mfma")
    tokens = case["q"].shape[0]
    cu = torch.tensor(case["host_cu"] + [tokens, tokens], dtype=torch.int32, device=DEV)
    table = torch.cat([case["block_table"], torch.zeros((2, case["block_table"].shape[1]), dtype=torch.int32, device=DEV)])
    scale = 1.0 / math.sqrt(head_dim)
    out = ops.paged_attention(
        case["q"], case["k_pages"], case["v_pages"], table, case["token_request"], case["positions"], cu, None,
        q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, scale=scale, window=window, max_seq_len=2048,
        v_transposed=case["v_transposed"])
    expected = _attention_expected(case, scale, window)
    assert np.abs(out.double().cpu().numpy() - expected).max() < _tol(dtype, 2)


@pytest.mark.parametrize("window", [None, 700])
def test_paged_attention_whole_long_prompts_many_tiles(window):
    """Whole prompts of a few thousand tokens beside a short one: dozens of tiles per head,
    more than fit on the GPU at once, so the order in which tiles are handed out (long and
    short ones paired) and the tile-to-request search over several requests are exercised."""
    q_heads, kv_heads, head_dim, page_size = 8, 2, 64, 16
    lengths = q_lens = [2210, 37, 300]
    case = _paged_case(torch.bfloat16, q_heads, kv_heads, head_dim, page_size, lengths, q_lens, seed=6,
                       v_transposed=True)
    out = _attend(case, q_heads, kv_heads, head_dim, 0.12, window, max(lengths))
    expected = _attention_expected(case, 0.12, window)
    assert np.abs(out.double().cpu().numpy() - expected).max() < _tol(torch.bfloat16, 2)


@pytest.mark.parametrize("q_heads,kv_heads,head_dim,page_size,window", [s for s in MFMA_SHAPES if s[2] <= 128])
@pytest.mark.parametrize("lengths,q_lens", [
    ([70, 33, 129, 64, 200], [70, 5, 1, 2, 37]),
    ([900, 37, 300], [900, 37, 300]),
    ([2500, 900, 700], [40, 3, 699]),
    ([1500, 17, 640, 300], [1, 1, 140, 90]),  # single tokens first: a launch of their own in the decode shape
])
def test_paged_attention_in_blocks_of_256_rows(monkeypatch, q_heads, kv_heads, head_dim, page_size, window, lengths, q_lens):
    """The launch shape that long prompts get (8 waves, 256 rows a block), forced here on
    short ones: mixed portions, whole prompts over many tiles, portions late in a long
    context (key ranges), groups of 1 to 20 heads; and the same through the usual shape."""
    from mini_infer_amd.ops import kernels

    case = _paged_case(torch.bfloat16, q_heads, kv_heads, head_dim, page_size, lengths, q_lens, seed=head_dim + 1,
                       v_transposed=True)
    scale = 1.0 / math.sqrt(head_dim)
    usual = _attend(case, q_heads, kv_heads, head_dim, scale, window, max(lengths))
    monkeypatch.setattr(kernels, "WIDE_PREFILL_MIN_BLOCKS", 1)
    shapes = []
    launch = kernels.library.load().mi_attn_mfma
    monkeypatch.setattr(kernels.library.load(), "mi_attn_mfma", lambda *a: (shapes.append(a[23]), launch(*a))[1])
    wide = _attend(case, q_heads, kv_heads, head_dim, scale, window, max(lengths))
    assert shapes == [kernels.ATTN_SHAPE_DECODE] * (q_lens[0] == 1) + [kernels.ATTN_SHAPE_PREFILL_WIDE]
    expected = _attention_expected(case, scale, window)
    assert np.abs(wide.double().cpu().numpy() - expected).max() < _tol(torch.bfloat16, 2)
    assert np.abs(usual.double().cpu().numpy() - expected).max() < _tol(torch.bfloat16, 2)


@pytest.mark.parametrize("rows_per_block", [128, 256])
@pytest.mark.parametrize("window", [None, 100])
def test_paged_attention_prompt_rows_find_planted_keys(monkeypatch, rows_per_block, window):
    """A whole prompt of 1,000 tokens in both prefill shapes: for chosen (query, key) pairs the
    key is made to stand out for that query, so the query's output must be that key's value.
    The pairs sit on the diagonal, at the first and last key, on both sides of the edges of the
    32-key tiles and of the 64- and 128-token row tiles, and on the window's edge; a tile that
    is skipped or masked wrongly, which random keys would hide in the tolerance, shows."""
    from mini_infer_amd.ops import kernels

    q_heads, kv_heads, head_dim, page_size, length = 2, 1, 64, 16, 1000
    scale = 1.0 / 8.0
    pairs = [(999, 0), (998, 998), (64, 64), (65, 63), (127, 96), (128, 127), (129, 129), (500, 31), (501, 32),
             (700, 255), (701, 256), (300, 201), (330, 300), (63, 2), (257, 254)]
    if window is not None:
        pairs = [(t, p) for t, p in pairs if t - p < window] + [(999, 900), (400, 301), (161, 62), (192, 93)]
    case = _paged_case(torch.bfloat16, q_heads, kv_heads, head_dim, page_size, [length], [length], seed=31,
                       v_transposed=True)
    assert len({p for _, p in pairs}) == len(pairs) == len({t for t, _ in pairs})
    for t, p in pairs:
        key = (case["qs"][0][t, 0].float() * 6.0).to(torch.bfloat16)  # score 6 |q|^2 / 8 = 48 +- a few
        case["ks"][0][p, 0] = key
        case["k_pages"][case["block_table"][0, p // page_size].item(), 0, p % page_size] = key.to(DEV)
    if rows_per_block == 256:
        monkeypatch.setattr(kernels, "WIDE_PREFILL_MIN_BLOCKS", 1)
    shapes = []
    launch = kernels.library.load().mi_attn_mfma
    monkeypatch.setattr(kernels.library.load(), "mi_attn_mfma", lambda *a: (shapes.append(a[23]), launch(*a))[1])
    out = _attend(case, q_heads, kv_heads, head_dim, scale, window, length)
    assert shapes == [kernels.ATTN_SHAPE_PREFILL_WIDE if rows_per_block == 256 else kernels.ATTN_SHAPE_PREFILL]
    out = out.float().cpu().reshape(length, q_heads, head_dim)
    for t, p in pairs:
        assert (out[t, 0] - case["vs"][0][p, 0].float()).abs().max() < 2e-2, (t, p)
    expected = _attention_expected(case, scale, window)
    assert np.abs(out.reshape(length, -1).double().numpy() - expected).max() < _tol(torch.bfloat16, 2)


@pytest.mark.parametrize("mode,dtype", ATTENTION_MODES)
def test_paged_attention_finds_one_far_key_and_respects_edges(mode, dtype):
    """One key among a thousand is made to stand out; the output must be its value.
    Placed at a page's first and last slot, at the causal edge and at the window's edge."""
    head_dim, page_size, length = 64, 16, 1000
    transposed = mode == "mfma"

    def plant(case, spot):
        q = case["qs"][0][0, 0].float()
        page = case["block_table"][0, spot // page_size].item()
        case["k_pages"][page, 0, spot % page_size] = (q * 4.0).to(dtype).to(DEV)  # score >> all others

    for window, spots in ((None, [0, 15, 16, 31, 32, 511, 512, 999]), (100, [900, 901, 911, 912, 927, 928, 999])):
        for spot in spots:
            case = _paged_case(dtype, 1, 1, head_dim, page_size, [length], [1], seed=spot, v_transposed=transposed)
            plant(case, spot)
            out = _attend(case, 1, 1, head_dim, 1.0, window, length)
            value = case["vs"][0][spot, 0].float()
            assert (out[0].float().cpu() - value).abs().max() < 2e-2, (window, spot)
    # a key just outside the window must not be seen, nor one after the query
    for spot, q_len in ((length - 100 - 1, 1), (length - 1, 2)):
        case = _paged_case(dtype, 1, 1, head_dim, page_size, [length], [q_len], seed=5, v_transposed=transposed)
        plant(case, spot)  # `ks` is not changed: the plain model never sees that key
        out = _attend(case, 1, 1, head_dim, 1.0, 100, length)
        expected = _attention_expected(case, 1.0, 100)
        rows = slice(0, 1)  # the first query (position length - q_len) must not see the planted key
        assert np.abs(out.double().cpu().numpy() - expected)[rows].max() < _tol(dtype, 2)


def test_paged_attention_long_context_in_many_key_ranges():
    """One token over 9,000 keys of one head: the matrix-core kernel cuts them into more
    ranges than for short contexts; a planted key in the first, a middle and the last
    range is found, and an unplanted case matches the plain model."""
    from mini_infer_amd import ops

    head_dim, page_size, length = 128, 16, 9000
    assert min(32, ops.attention_splits(1, length, target=256, min_keys=128)) == 32
    for spot in (3, 4500, 8999):
        case = _paged_case(torch.bfloat16, 4, 1, head_dim, page_size, [length], [1], seed=spot, v_transposed=True)
        q = case["qs"][0][0, 2].float()  # the third of the four heads that share the keys
        page = case["block_table"][0, spot // page_size].item()
        case["k_pages"][page, 0, spot % page_size] = (q * 2.0).bfloat16().to(DEV)
        out = _attend(case, 4, 1, head_dim, 1.0, None, length)
        value = case["vs"][0][spot, 0].float()
        assert (out[0, 2 * head_dim : 3 * head_dim].float().cpu() - value).abs().max() < 2e-2, spot
    case = _paged_case(torch.bfloat16, 4, 1, head_dim, page_size, [length], [1], seed=11, v_transposed=True)
    out = _attend(case, 4, 1, head_dim, 0.05, None, length)
    expected = _attention_expected(case, 0.05, None)
    assert np.abs(out.double().cpu().numpy() - expected).max() < _tol(torch.bfloat16, 2)


@pytest.mark.parametrize(
    "q_heads,kv_heads,head_dim,lengths",
    [(32, 8, 128, [3000]), (6, 2, 64, [700, 2049]), (3, 1, 32, [517]), (32, 8, 128, [2100, 2500, 3000, 2048, 4000, 2222, 3100, 2900]),
     (6, 2, 64, [700, 2049, 333, 900, 1200, 800, 650, 1500, 400, 512, 2000])],
)
def test_output_projection_from_uncombined_key_ranges(q_heads, kv_heads, head_dim, lengths):
    """A few single tokens: the attention leaves its key ranges uncombined and the output
    projection combines them on its way; the same numbers as combining first."""
    from mini_infer_amd import ops

    case = _paged_case(torch.bfloat16, q_heads, kv_heads, head_dim, 16, lengths, [1] * len(lengths), seed=41,
                       v_transposed=True)
    args = (case["q"], case["k_pages"], case["v_pages"], case["block_table"], case["token_request"],
            case["positions"], case["cu"], case["host_cu"])
    kwargs = dict(q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, scale=0.3, window=None,
                  max_seq_len=max(lengths), v_transposed=True)
    whole = ops.paged_attention(*args, **kwargs)
    pieces = ops.paged_attention(*args, **kwargs, combine=False)
    assert ops.attention_pieces_pay(1, q_heads, head_dim)
    assert isinstance(pieces, ops.AttentionPieces) and pieces.splits > 1 and pieces.tokens == len(lengths)
    assert (pieces.finish().float() - whole.float()).abs().max() < 2e-2
    for n in (q_heads * head_dim, 1000, 24):
        w = _rand(n, q_heads * head_dim, dtype=torch.bfloat16, seed=42, scale=0.1)
        assert torch.equal(ops.linear_from_attention(pieces, w), ops.linear(whole, w))
    # with nothing to combine, or more than single tokens, the attention comes back whole
    short = _paged_case(torch.bfloat16, q_heads, kv_heads, head_dim, 16, [40], [1], seed=43, v_transposed=True)
    out = ops.paged_attention(short["q"], short["k_pages"], short["v_pages"], short["block_table"], short["token_request"],
                              short["positions"], short["cu"], short["host_cu"], q_heads=q_heads, kv_heads=kv_heads,
                              head_dim=head_dim, scale=0.3, window=None, max_seq_len=40, v_transposed=True, combine=False)
    assert isinstance(out, torch.Tensor)
    assert not ops.attention_pieces_pay(2, 32, 128) and not ops.attention_pieces_pay(1, 4, 48)


@pytest.mark.parametrize(
    "m,n,k,inter",
    [(8, 4096, 4096, 14336), (1, 4096, 4096, 14336), (16, 96, 64, 160), (7, 160, 96, 301), (13, 4128, 160, 40), (3, 32, 32, 5),
     (6, 1536, 1536, 520), (5, 1000, 512, 72), (16, 8200, 1024, 24)],
)
def test_product_add_and_norm_folded_into_two_products(m, n, k, inter):
    """`linear_add_norm` (product, add into the residual, norm but for the rows' factors) followed
    by `linear_swiglu` on its `ScaledRows`, against the four kernels they replace and against
    float64: the residual is bit-equal (the same rounded product added in float32), the
    activations agree as two bfloat16 roundings of the same numbers do."""
    from mini_infer_amd import ops

    x = _rand(m, k, dtype=torch.bfloat16, seed=51)
    w = _rand(n, k, dtype=torch.bfloat16, seed=52, scale=0.1)
    norm_w = (torch.rand(n, generator=torch.Generator().manual_seed(53)) + 0.5).bfloat16().to(DEV)
    gate_up = _rand(2 * inter, n, dtype=torch.bfloat16, seed=54, scale=0.08)
    residual0 = _rand(m, n, dtype=torch.float32, seed=55)
    eps = 3e-5

    apart_residual = residual0.clone()
    normed = ops.add_rmsnorm(ops.linear(x, w), apart_residual, norm_w, eps)
    apart = ops.linear_swiglu(normed, gate_up)

    residual = residual0.clone()
    rows = ops.linear_add_norm(ops.PendingProduct(x, w), residual, norm_w, eps)
    assert isinstance(rows, ops.ScaledRows) and rows.values.shape == (m, n) and rows.sumsq.shape[1] == m
    assert torch.equal(residual, apart_residual)
    # the pieces add up to the rows' sums of squares, and finish() is the norm's output
    exact_sumsq = (residual.double() ** 2).sum(dim=1)
    assert ((rows.sumsq.double().sum(dim=0) - exact_sumsq).abs() <= 1e-5 * exact_sumsq).all()
    exact_normed = residual.double() * torch.rsqrt(exact_sumsq / n + eps)[:, None] * norm_w.double()
    assert (rows.finish().double() - exact_normed).abs().max() < 2.0 ** -6 * float(exact_normed.abs().max())
    folded = ops.linear_swiglu(rows, gate_up)
    assert folded.shape == (m, inter)
    residual_off = residual0.clone()
    rows_off = ops.linear_add_norm(ops.PendingProduct(x, _off_the_cache_lines(w)), residual_off, norm_w, eps)
    assert torch.equal(residual_off, residual) and torch.equal(rows_off.values, rows.values)
    assert torch.equal(rows_off.sumsq, rows.sumsq)
    assert torch.equal(ops.linear_swiglu(rows, _off_the_cache_lines(gate_up)), folded)

    def activation(normed_rows):
        both = (normed_rows @ gate_up.double().T).bfloat16().double()
        return both[:, :inter] / (1 + torch.exp(-both[:, :inter])) * both[:, inter:]

    exact = activation(exact_normed)
    bound = 2.0 ** -5 * float(exact.abs().max()) + 1e-6
    assert (folded.double() - exact).abs().max() < bound
    assert (apart.double() - exact).abs().max() < bound  # (the yardstick: the four kernels are no closer)
    # rows that meet something else than that product are finished first: the same function
    assert ops.linear_swiglu(ops.ScaledRows(rows.values.float(), rows.sumsq, eps), gate_up.float()).shape == (m, inter)


@pytest.mark.parametrize("q_heads,kv_heads,head_dim,lengths", [(32, 8, 128, [3000]), (6, 2, 64, [700]), (3, 1, 32, [517])])
def test_product_add_and_norm_from_uncombined_key_ranges(q_heads, kv_heads, head_dim, lengths):
    """The same fold with a single token's attention still in its key ranges: what
    `linear_from_attention` then `add_rmsnorm` give, bit for bit in the residual."""
    from mini_infer_amd import ops

    case = _paged_case(torch.bfloat16, q_heads, kv_heads, head_dim, 16, lengths, [1] * len(lengths), seed=61,
                       v_transposed=True)
    pieces = ops.paged_attention(
        case["q"], case["k_pages"], case["v_pages"], case["block_table"], case["token_request"], case["positions"],
        case["cu"], case["host_cu"], q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, scale=0.3, window=None,
        max_seq_len=max(lengths), v_transposed=True, combine=False)
    assert isinstance(pieces, ops.AttentionPieces)
    k, n = q_heads * head_dim, 4096 if head_dim == 128 else 200
    w = _rand(n, k, dtype=torch.bfloat16, seed=62, scale=0.1)
    norm_w = (torch.rand(n, generator=torch.Generator().manual_seed(63)) + 0.5).bfloat16().to(DEV)
    residual0 = _rand(len(lengths), n, dtype=torch.float32, seed=64)
    apart_residual, residual = residual0.clone(), residual0.clone()
    normed = ops.add_rmsnorm(ops.linear_from_attention(pieces, w), apart_residual, norm_w, 1e-5)
    rows = ops.linear_add_norm(ops.PendingProduct(pieces, w), residual, norm_w, 1e-5)
    assert torch.equal(residual, apart_residual)
    assert (rows.finish().float() - normed.float()).abs().max() <= 2.0 ** -6 * float(normed.float().abs().max())


@pytest.mark.parametrize("v_transposed", [False, True])
@pytest.mark.parametrize(
    "m,inter,hidden,q_heads,kv_heads,head_dim",
    [(8, 14336, 4096, 32, 8, 128), (1, 14336, 4096, 32, 8, 128), (16, 160, 96, 3, 1, 32), (5, 320, 160, 6, 2, 64), (3, 1536, 1536, 6, 2, 64)],
)
def test_down_product_add_and_norm_folded_into_the_next_q_k_v_product(v_transposed, m, inter, hidden, q_heads, kv_heads, head_dim):
    """`linear_add_norm` on a feed-forward's last product, then `qkv_rope_write` on its
    `ScaledRows`, against the three kernels they replace (product, add + norm, q|k|v with
    rotation and cache write): the residual bit for bit, queries, keys and values as two
    bfloat16 roundings of the same numbers agree, and against float64."""
    from mini_infer_amd import ops

    page_size, num_pages = 16, 5
    width = (q_heads + 2 * kv_heads) * head_dim
    act = _rand(m, inter, dtype=torch.bfloat16, seed=71)
    down = _rand(hidden, inter, dtype=torch.bfloat16, seed=72, scale=0.05)
    norm_w = (torch.rand(hidden, generator=torch.Generator().manual_seed(73)) + 0.5).bfloat16().to(DEV)
    qkv_w = _rand(width, hidden, dtype=torch.bfloat16, seed=74, scale=0.1)
    residual0 = _rand(m, hidden, dtype=torch.float32, seed=75)
    positions = torch.tensor([0, 1, 700, 5, 131071, 17, 18, 19, 3000, 2, 4, 6, 8, 10, 12, 14][:m], dtype=torch.int32, device=DEV)
    cos, sin = ops.rope_table(positions, torch.from_numpy(pl.inv_freq_default(head_dim, 500000.0)).to(DEV))
    slots = torch.tensor([40, 3, 17, 16, 0, 43, -1, 9, 22, 5, 6, 7, 30, 31, 32, 33][:m], dtype=torch.int32, device=DEV)
    eps = 2e-5

    def pages():
        k = torch.full((num_pages, kv_heads, page_size, head_dim), 7.0, dtype=torch.bfloat16, device=DEV)
        v_shape = (num_pages, kv_heads, head_dim, page_size) if v_transposed else k.shape
        return k, torch.full(v_shape, 7.0, dtype=torch.bfloat16, device=DEV)

    heads = dict(q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, v_transposed=v_transposed)
    apart_residual = residual0.clone()
    normed = ops.add_rmsnorm(ops.linear(act, down), apart_residual, norm_w, eps)
    k_apart, v_apart = pages()
    q_apart = ops.qkv_rope_write(normed, qkv_w, cos, sin, slots, k_apart, v_apart, **heads)

    residual = residual0.clone()
    rows = ops.linear_add_norm(ops.PendingProduct(act, down), residual, norm_w, eps)
    assert torch.equal(residual, apart_residual)
    assert ops.qkv_rope_write_takes(rows, qkv_w, head_dim, head_dim, False)
    k_fold, v_fold = pages()
    q_fold = ops.qkv_rope_write(rows, qkv_w, cos, sin, slots, k_fold, v_fold, **heads)

    # float64: the norm of the float32 residual the kernels left, the product rounded once, the rotation
    exact_sumsq = (residual.double() ** 2).sum(dim=1)
    exact_normed = residual.double() * torch.rsqrt(exact_sumsq / hidden + eps)[:, None] * norm_w.double()
    qkv = (exact_normed @ qkv_w.double().T).bfloat16().double().view(m, q_heads + 2 * kv_heads, head_dim)
    half = head_dim // 2
    c, s_ = cos.double()[:, None, :], sin.double()[:, None, :]
    rotated = torch.cat([qkv[..., :half] * c - qkv[..., half:] * s_, qkv[..., half:] * c + qkv[..., :half] * s_], dim=-1)
    exact_q = rotated[:, :q_heads].reshape(m, q_heads * head_dim)
    bound = 2.0 ** -5 * float(exact_q.abs().max()) + 1e-6
    assert (q_fold.double() - exact_q).abs().max() < bound
    assert (q_apart.double() - exact_q).abs().max() < bound  # (the yardstick: the three kernels are no closer)
    for row in range(m):
        slot = int(slots[row])
        if slot < 0:
            continue
        page, off = divmod(slot % (num_pages * page_size), page_size)
        exact_k = rotated[row, q_heads : q_heads + kv_heads]
        exact_v = qkv[row, q_heads + kv_heads :]
        got_v = v_fold[page, :, :, off] if v_transposed else v_fold[page, :, off]
        assert (k_fold[page, :, off].double() - exact_k).abs().max() < bound
        assert (got_v.double() - exact_v).abs().max() < bound
    # slots nobody wrote keep what they held, in both ways of running
    written = torch.zeros(num_pages * page_size, dtype=torch.bool, device=DEV)
    written[slots[slots >= 0].long()] = True
    untouched = ~written.view(num_pages, page_size)
    assert torch.all(k_fold.permute(0, 2, 1, 3)[untouched] == 7.0) and torch.all(k_apart.permute(0, 2, 1, 3)[untouched] == 7.0)
    # rows that meet a product without such a kernel are finished first: the same function
    many = ops.ScaledRows(rows.values.float(), rows.sumsq, eps)
    assert not ops.qkv_rope_write_takes(many, qkv_w.float(), head_dim, head_dim, False)


def test_kernels_refuse_what_they_do_not_take():
    from mini_infer_amd import ops
    from mini_infer_amd.exceptions import KernelShapeError

    for head_dim, message in ((25, "even"), (258, "at most 256")):
        case = _paged_case(torch.float32, 4, 2, head_dim, 4, [5], [1])
        with pytest.raises(KernelShapeError, match=message):
            _attend(case, 4, 2, head_dim, 1.0, None, 5)
    # transposed value pages belong to the matrix-core kernel, which takes bfloat16 only
    case = _paged_case(torch.float32, 4, 2, 32, 16, [5], [1], v_transposed=True)
    with pytest.raises(KernelShapeError, match="matrix-core"):
        _attend(case, 4, 2, 32, 1.0, None, 5)
    assert ops.mfma_attention_supported(torch.bfloat16, 128, 16)
    assert not ops.mfma_attention_supported(torch.bfloat16, 48, 16)
    assert not ops.mfma_attention_supported(torch.bfloat16, 128, 8)
    assert not ops.mfma_attention_supported(torch.float32, 128, 16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.silu_mul(torch.zeros(2, 8))
    with pytest.raises(KernelShapeError):
        ops.add_rmsnorm(None, torch.zeros(2, 8, device=DEV), torch.ones(9, device=DEV), 1e-5)
    with pytest.raises(KernelShapeError):
        ops.gemm_f32(torch.zeros(2, 8, device=DEV), torch.zeros(3, 9, device=DEV))
