"""The entry point that allocates nothing (decode attention over a file-scope scratch array),
called through ctypes as a caller without torch bindings would, against the existing entry point
that takes its workspace as arguments."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

RUN_KEYS = 256


def _case(seed, n_tokens, nh, nkv, hd, page_size, contexts, window_kind=0, window=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    dev = "cuda:0"
    blocks = [(c + page_size - 1) // page_size for c in contexts]
    maxb = max(blocks)
    num_pages = sum(blocks) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    table = torch.full((n_tokens, maxb), -1, dtype=torch.int32)
    o = 0
    for i, b in enumerate(blocks):
        table[i, :b] = torch.tensor(perm[o:o + b], dtype=torch.int32)
        o += b
    k = (torch.randn(num_pages, nkv, page_size, hd, generator=g) * 0.5).to(torch.bfloat16)
    v = (torch.randn(num_pages, nkv, hd, page_size, generator=g) * 0.5).to(torch.bfloat16)
    q = torch.randn(n_tokens, nh * hd, generator=g).to(torch.bfloat16)
    pos = torch.tensor([c - 1 for c in contexts], dtype=torch.int32)
    ent = torch.arange(n_tokens, dtype=torch.int32)
    max_ctx = max(contexts)
    max_splits = ((max_ctx - 1) >> 4) // (RUN_KEYS // 16) + 1
    return dict(q=q.to(dev), k=k.to(dev), v=v.to(dev), table=table.to(dev), pos=pos.to(dev), ent=ent.to(dev),
                n=n_tokens, nh=nh, nkv=nkv, hd=hd, ps=page_size, maxb=maxb, pages=num_pages, splits=max_splits,
                wk=window_kind, w=window, scale=1.0 / math.sqrt(hd))


def _both(lib, c):
    """(existing entry point's output, the new one's) for one case."""
    P, I, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    old = lib.sharpi_attention_decode
    old.argtypes = [P] * 10 + [I, I, F] + [I] * 8 + [P]
    old.restype = I
    new = lib.sharpi_attention_decode_noalloc
    new.argtypes = [P] * 8 + [I, I, F] + [I] * 8 + [P]
    new.restype = I
    stream = torch.cuda.current_stream().cuda_stream
    part_o = torch.empty(c["n"] * c["nh"] * c["splits"] * c["hd"], dtype=torch.float32, device="cuda:0")
    part_ml = torch.empty(c["n"] * c["nh"] * c["splits"] * 2, dtype=torch.float32, device="cuda:0")
    out_old = torch.zeros_like(c["q"])
    out_new = torch.zeros_like(c["q"])
    tail = (c["wk"], c["w"], c["scale"], c["n"], c["nh"], c["nkv"], c["hd"], c["ps"], c["maxb"], c["pages"], c["splits"], stream)
    head = (c["q"].data_ptr(), c["k"].data_ptr(), c["v"].data_ptr(), c["table"].data_ptr(), c["ent"].data_ptr(),
            c["pos"].data_ptr(), None)
    rc = old(*head, part_o.data_ptr(), part_ml.data_ptr(), out_old.data_ptr(), *tail)
    assert rc == 0, rc
    rc = new(*head, out_new.data_ptr(), *tail)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return out_old, out_new


def test_decode_attention_without_allocation_equals_the_workspace_form():
    from sharpinference_amd.ops import lib as kernel_lib

    lib = kernel_lib.load()
    # two calls in a row on the same scratch array, the second smaller (fewer tokens, shorter
    # contexts, fewer runs): what the first left behind must not leak into the second
    first = _case(1, n_tokens=7, nh=10, nkv=2, hd=128, page_size=16, contexts=[700, 3, 257, 256, 1024, 33, 512])
    second = _case(2, n_tokens=3, nh=10, nkv=2, hd=128, page_size=16, contexts=[40, 300, 17])
    third = _case(3, n_tokens=4, nh=6, nkv=3, hd=64, page_size=32, contexts=[90, 500, 64, 129], window_kind=1, window=96)
    for c in (first, second, third):
        a, b = _both(lib, c)
        assert torch.isfinite(a.float()).all()
        assert float(a.float().abs().max()) > 0
        assert torch.equal(a, b)


def test_a_bound_on_the_runs_that_is_too_small_shows_as_nan_not_as_wrong_attention():
    """A caller of either entry point that passes fewer runs than a token's keys span would lose
    the keys nearest the query: such a token's row comes back as NaN, the others' rows as they are."""
    from sharpinference_amd.ops import lib as kernel_lib

    lib = kernel_lib.load()
    c = _case(4, n_tokens=3, nh=10, nkv=2, hd=128, page_size=16, contexts=[200, 700, 256])
    good_old, good_new = _both(lib, c)
    assert torch.equal(good_old, good_new) and torch.isfinite(good_old.float()).all()
    c["splits"] = 1                       # enough for 256 keys: tokens 0 and 2, not token 1
    bad_old, bad_new = _both(lib, c)
    for bad in (bad_old, bad_new):
        assert torch.isnan(bad[1].float()).all()
        assert torch.equal(bad[0], good_old[0]) and torch.equal(bad[2], good_old[2])


def test_sizes_beyond_the_scratch_array_are_refused():
    from sharpinference_amd.ops import lib as kernel_lib

    lib = kernel_lib.load()
    P, I, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    new = lib.sharpi_attention_decode_noalloc
    new.argtypes = [P] * 8 + [I, I, F] + [I] * 8 + [P]
    new.restype = I
    # 4,096 tokens x 64 heads x 16 runs x 130 floats is far beyond 8 Mi floats: refused on the host, nothing launched
    rc = new(None, None, None, None, None, None, None, None, 0, 0, 1.0, 4096, 64, 8, 128, 16, 256, 1024, 16, None)
    assert rc == 1001
