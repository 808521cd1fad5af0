"""The attention entry point that allocates nothing, called through ctypes as a foreign
caller would, against the entry point that takes its partial buffers from the caller.

Two calls in a row on the same GPU, the second with a smaller input: the library's own
array still holds the first call's partial results then, and none of them may leak into
the second result.  Both entry points run the same kernels in the same order, so the
outputs must agree bit for bit; the first is also compared with a plain attention in
float64.  That nothing is allocated is checked where it can be: the device's free memory
is the same before and after the calls, and a call records into a HIP graph (a stream
that records refuses every allocation) whose replays give the eager result.
"""

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
_P = c_void_p
SCRATCH_BYTES = 8 << 20


def _library():
    from mini_infer_amd.ops import library

    library.load()
    lib = ctypes.CDLL(str(library.library_path()))
    lib.mi_last_error.restype = ctypes.c_char_p
    lib.mi_attn_generic_static.restype = c_int
    lib.mi_attn_generic_static.argtypes = [
        c_int, _P, c_int64, _P, _P, _P, c_int, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int,
        c_int, c_float, c_int, c_int, _P, _P,
    ]
    lib.mi_attn_generic.restype = c_int
    lib.mi_attn_generic.argtypes = [
        c_int, _P, c_int64, _P, _P, _P, c_int, _P, _P, _P, c_int64, _P, _P, c_int, c_int, c_int,
        c_int, c_int, c_int, c_float, c_int, c_int, _P, _P,
    ]
    return lib


def _case(dtype, q_heads, kv_heads, head_dim, page_size, lengths, seed):
    """Single-token queries at the end of contexts of the given lengths, pages shuffled."""
    rng = np.random.default_rng(seed)
    pages_per = [-(-n // page_size) for n in lengths]
    num_pages = sum(pages_per) + 2
    order = rng.permutation(num_pages).astype(np.int32)
    table = np.full((len(lengths), max(pages_per)), -1, dtype=np.int32)
    at = 0
    for b, count in enumerate(pages_per):
        table[b, :count] = order[at : at + count]
        at += count
    make = lambda *shape: torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to(dtype).to(DEV)  # noqa: E731
    return dict(
        q=make(len(lengths), q_heads * head_dim),
        k_pages=make(num_pages, kv_heads, page_size, head_dim),
        v_pages=make(num_pages, kv_heads, page_size, head_dim),
        table=torch.from_numpy(table).to(DEV),
        token_request=torch.arange(len(lengths), dtype=torch.int32, device=DEV),
        positions=torch.tensor([n - 1 for n in lengths], dtype=torch.int32, device=DEV),
        sizes=(len(lengths), q_heads, kv_heads, head_dim, page_size, num_pages),
    )


def _run(lib, case, dtype, splits, static, window=0):
    tokens, q_heads, kv_heads, head_dim, page_size, num_pages = case["sizes"]
    out = torch.full((tokens, q_heads * head_dim), float("nan"), dtype=dtype, device=DEV)
    code = 0 if dtype == torch.float32 else 1
    stream = torch.cuda.current_stream().cuda_stream
    common = (code, case["q"].data_ptr(), q_heads * head_dim, case["k_pages"].data_ptr(), case["v_pages"].data_ptr(),
              case["table"].data_ptr(), case["table"].shape[1], case["token_request"].data_ptr(),
              case["positions"].data_ptr(), out.data_ptr(), q_heads * head_dim)
    tail = (tokens, q_heads, kv_heads, head_dim, page_size, num_pages, 0.17, window, splits, None, stream)
    if static:
        status = lib.mi_attn_generic_static(*common, *tail)
    else:
        acc = torch.empty(tokens * q_heads * splits * head_dim, dtype=torch.float32, device=DEV)
        ml = torch.empty(tokens * q_heads * splits * 2, dtype=torch.float32, device=DEV)
        status = lib.mi_attn_generic(*common, acc.data_ptr(), ml.data_ptr(), *tail)
    torch.cuda.synchronize()
    return status, out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_calls_in_a_row_the_second_smaller_equal_the_allocating_entry_point(dtype):
    lib = _library()
    large = _case(dtype, q_heads=12, kv_heads=3, head_dim=80, page_size=16, lengths=[700, 333, 64, 1029, 5], seed=1)
    small = _case(dtype, q_heads=4, kv_heads=2, head_dim=48, page_size=8, lengths=[90, 17], seed=2)
    for case, splits in ((large, 7), (small, 3)):
        status, expected = _run(lib, case, dtype, splits, static=False)
        assert status == 0, lib.mi_last_error()
        status, got = _run(lib, case, dtype, splits, static=True)
        assert status == 0, lib.mi_last_error()
        assert not torch.isnan(got).any()
        assert torch.equal(got, expected)
    # and the large one again after the small one
    status, expected = _run(lib, large, dtype, 7, static=False)
    status, got = _run(lib, large, dtype, 7, static=True)
    assert status == 0 and torch.equal(got, expected)
    # one key range: the library's array is not touched at all
    status, expected = _run(lib, small, dtype, 1, static=False)
    status, got = _run(lib, small, dtype, 1, static=True)
    assert status == 0 and torch.equal(got, expected)


def test_what_does_not_fit_the_librarys_array_is_refused_and_nothing_runs():
    lib = _library()
    case = _case(torch.float32, q_heads=32, kv_heads=8, head_dim=128, page_size=16, lengths=[40] * 64, seed=3)
    tokens, q_heads, _, head_dim, _, _ = case["sizes"]
    splits = 16
    assert tokens * q_heads * splits * (head_dim + 2) * 4 > SCRATCH_BYTES
    status, out = _run(lib, case, torch.float32, splits, static=True)
    assert status != 0 and b"bytes" in lib.mi_last_error()
    assert torch.isnan(out).all()  # the output was never written
    status, out = _run(lib, case, torch.float32, 3, static=True)  # fewer ranges fit
    assert status == 0 and not torch.isnan(out).any()


def _plain_attention(case, scale):
    """Every token's attention over its own context, in float64 (single-token queries)."""
    tokens, q_heads, kv_heads, head_dim, page_size, _ = case["sizes"]
    q = case["q"].double().cpu().reshape(tokens, q_heads, head_dim)
    k_pages, v_pages = case["k_pages"].double().cpu(), case["v_pages"].double().cpu()
    table, positions = case["table"].cpu(), case["positions"].cpu()
    out = torch.zeros(tokens, q_heads, head_dim, dtype=torch.float64)
    for t in range(tokens):
        n = int(positions[t]) + 1
        pages = table[t, : -(-n // page_size)].long()
        k = k_pages[pages].permute(1, 0, 2, 3).reshape(kv_heads, -1, head_dim)[:, :n]
        v = v_pages[pages].permute(1, 0, 2, 3).reshape(kv_heads, -1, head_dim)[:, :n]
        for h in range(q_heads):
            weights = torch.softmax((k[h // (q_heads // kv_heads)] @ q[t, h]) * scale, dim=0)
            out[t, h] = weights @ v[h // (q_heads // kv_heads)]
    return out.reshape(tokens, q_heads * head_dim)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_entry_point_that_allocates_nothing_against_a_plain_attention(dtype):
    lib = _library()
    case = _case(dtype, q_heads=6, kv_heads=2, head_dim=40, page_size=8, lengths=[130, 7, 61], seed=4)
    status, got = _run(lib, case, dtype, 4, static=True)
    assert status == 0, lib.mi_last_error()
    expected = _plain_attention(case, 0.17)
    assert float((got.double().cpu() - expected).abs().max()) < (2e-5 if dtype == torch.float32 else 2e-2)


def test_free_memory_is_unchanged_and_a_call_records_into_a_graph():
    lib = _library()
    dtype = torch.float32
    case = _case(dtype, q_heads=8, kv_heads=2, head_dim=64, page_size=16, lengths=[400, 90, 257], seed=5)
    tokens, q_heads, kv_heads, head_dim, page_size, num_pages = case["sizes"]
    out = torch.zeros((tokens, q_heads * head_dim), dtype=dtype, device=DEV)

    def call(stream):
        return lib.mi_attn_generic_static(
            0, case["q"].data_ptr(), q_heads * head_dim, case["k_pages"].data_ptr(), case["v_pages"].data_ptr(),
            case["table"].data_ptr(), case["table"].shape[1], case["token_request"].data_ptr(),
            case["positions"].data_ptr(), out.data_ptr(), q_heads * head_dim, tokens, q_heads, kv_heads, head_dim,
            page_size, num_pages, 0.17, 0, 5, None, stream)

    assert call(torch.cuda.current_stream().cuda_stream) == 0  # (the first call asks for the array's address)
    torch.cuda.synchronize()
    eager = out.clone()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        assert call(torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    # recorded: an allocation (or a free) while a stream records is an error, and there is none
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        status = call(torch.cuda.current_stream().cuda_stream)
    assert status == 0, lib.mi_last_error()
    for replay in range(3):
        out.zero_()
        case["q"].add_(0.0)  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay}"
