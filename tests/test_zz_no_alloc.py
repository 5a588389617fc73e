"""The attention entry point that allocates nothing (``ni_token_attention_static``), called through
``ctypes`` as a caller outside this package would, against the entry point that takes the caller's
workspace (``ni_token_attention``): two calls in a row, the second with a smaller input, which
finds the first call's partial results still in the library's own array."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

HD, H, KVH, PAGE = 64, 8, 2, 16


def _library():
    from nanoinfer_amd.csrc import build
    name, sources, defines = build.attention_target(HD)
    lib = ctypes.CDLL(build.library_path(name, sources, defines))
    lib.ni_token_attention_static_floats.restype = ctypes.c_long
    return lib


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _case(n_tokens, context, nsplit, dtype, seed):
    """``n_tokens`` single tokens of as many sequences, each at the end of ``context`` keys, with
    pages dealt out in a shuffled order."""
    g = torch.Generator().manual_seed(seed)
    dev = torch.device("cuda", 0)
    pages_per_seq = (context + PAGE - 1) // PAGE
    n_pages = n_tokens * pages_per_seq + 3
    q = torch.randn(n_tokens, H * HD, generator=g).to(dev, dtype)
    kpool = torch.randn(n_pages, KVH, PAGE, HD, generator=g).to(dev, dtype)
    vpool = torch.randn(n_pages, KVH, PAGE, HD, generator=g).to(dev, dtype)
    ids = torch.randperm(n_pages, generator=g)[: n_tokens * pages_per_seq].to(torch.int32)
    table = ids.view(n_tokens, pages_per_seq).contiguous().to(dev)
    seq = torch.arange(n_tokens, dtype=torch.int32, device=dev)
    pos = torch.tensor([context - 1 - 3 * i for i in range(n_tokens)], dtype=torch.int32, device=dev)
    return q, kpool, vpool, table, seq, pos


def _both(lib, n_tokens, context, nsplit, dtype, seed):
    q, kpool, vpool, table, seq, pos = _case(n_tokens, context, nsplit, dtype, seed)
    code = 0 if dtype == torch.float32 else 1
    scale = ctypes.c_float(1.0 / math.sqrt(HD))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    want = torch.empty(n_tokens, H * HD, dtype=dtype, device=q.device)
    got = torch.full_like(want, float("nan"))
    rows = n_tokens * H * nsplit
    work = torch.empty(rows * (HD + 2), dtype=torch.float32, device=q.device)
    part_o, part_ml = work[: rows * HD], work[rows * HD:]
    err = lib.ni_token_attention(_ptr(q), H * HD, _ptr(kpool), _ptr(vpool), _ptr(table), table.shape[1], _ptr(seq),
                                 _ptr(pos), _ptr(want), _ptr(part_o), _ptr(part_ml), n_tokens, H, KVH, PAGE, 0, scale,
                                 nsplit, code, stream)
    assert err == 0
    torch.cuda.synchronize()

    def static_call(out):
        return lib.ni_token_attention_static(_ptr(q), H * HD, _ptr(kpool), _ptr(vpool), _ptr(table), table.shape[1],
                                             _ptr(seq), _ptr(pos), _ptr(out), n_tokens, H, KVH, PAGE, 0, scale, nsplit,
                                             code, stream)

    # once first: the library's code object and its array come to the device with its first launch.  From
    # then on a call must leave both the framework's allocator and the driver's count of free device
    # memory where they were (the latter sees a hipMalloc that the former never hears of).
    first = torch.full_like(want, float("nan"))
    assert static_call(first) == 0
    torch.cuda.synchronize()
    held, free = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    assert static_call(got) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == held
    assert torch.cuda.mem_get_info()[0] == free, "device memory was taken or given back during the call"
    assert torch.equal(first, got)
    assert bool(torch.isfinite(got.float()).all())
    assert torch.equal(got, want), float((got.float() - want.float()).abs().max())
    return got


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_calls_in_a_row_the_second_smaller(dtype):
    lib = _library()
    _both(lib, n_tokens=6, context=700, nsplit=5, dtype=dtype, seed=1)
    _both(lib, n_tokens=2, context=300, nsplit=3, dtype=dtype, seed=2)      # finds the first call's leftovers
    _both(lib, n_tokens=3, context=90, nsplit=1, dtype=dtype, seed=3)       # no runs: the array is not touched


def test_more_than_the_array_holds_is_refused():
    lib = _library()
    cap = lib.ni_token_attention_static_floats()
    assert cap == 1 << 20
    n_tokens, nsplit = 64, 40
    assert n_tokens * H * nsplit * (HD + 2) > cap
    q, kpool, vpool, table, seq, pos = _case(n_tokens, 256, nsplit, torch.float32, 4)
    out = torch.zeros(n_tokens, H * HD, device=q.device)
    err = lib.ni_token_attention_static(_ptr(q), H * HD, _ptr(kpool), _ptr(vpool), _ptr(table), table.shape[1],
                                        _ptr(seq), _ptr(pos), _ptr(out), n_tokens, H, KVH, PAGE, 0,
                                        ctypes.c_float(0.125), nsplit, 0,
                                        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert err == -3
    assert float(out.abs().max()) == 0.0          # nothing was launched
