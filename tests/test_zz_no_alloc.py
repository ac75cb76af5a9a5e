"""The decode attention's entry point that allocates nothing (llogos_attn_decode_static_bf16),
called through ctypes as a caller outside the package would: its output must equal, bit for
bit, that of llogos_attn_decode_bf16 with a workspace from the caller, on two calls in a row
of which the second is smaller (the library's one scratch array keeps the first call's
contents), and a step that needs more scratch than the array holds must be refused.  One
case has a window and sinks, with the page-table entries of pages outside the window at -1
(their blocks write empty partial results over what the larger call before left), and every
case is also compared with a plain attention in float64 over the same pages."""
import ctypes
import importlib
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
library = importlib.import_module("daisi-llogos_amd.ops.library")
DEV = "cuda:0"
P, I, F, LL = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong


def _lib():
    lib = library.load()
    lib.llogos_attn_decode_static_bf16.argtypes = [P, P, I, P, P, P, I, I, P, I, I, I, I, F, I, I, P]
    lib.llogos_attn_decode_static_bf16.restype = I
    lib.llogos_attn_decode_bf16.argtypes = [P, P, I, P, P, P, I, I, P, I, I, I, I, F, I, I, P, LL, P]
    lib.llogos_attn_decode_bf16.restype = I
    lib.llogos_attn_decode_workspace.argtypes = [I, I, I, I, I]
    lib.llogos_attn_decode_workspace.restype = LL
    lib.llogos_attn_decode_static_capacity.restype = LL
    lib.llogos_attn_decode_static_init.restype = I
    return lib


def _visible(q_pos, k_pos, window, sinks):
    return k_pos <= q_pos and (window <= 0 or k_pos < sinks or k_pos > q_pos - window)


def _plain(q, kp, vp, table, pos, nh, nkv, hd, window, sinks):
    """softmax(q . K^T / sqrt(hd)) . V per head in float64, keys and values taken from the pages by the
    cache's own rule for where a (token, dimension) lies in a page."""
    pages = importlib.import_module("daisi-llogos_amd.cache.pages")
    ki, vi = (torch.tensor(x) for x in pages.page_offsets(hd))         # [64, hd] element offsets
    q, kp, vp, table, pos = (t.cpu() for t in (q, kp, vp, table, pos))
    out = torch.zeros((q.shape[0], nh * hd), dtype=torch.float64)
    for b in range(q.shape[0]):
        seen = [t for t in range(int(pos[b]) + 1) if _visible(int(pos[b]), t, window, sinks)]
        page, at = table[b].long()[torch.tensor(seen) // 64], torch.tensor(seen) % 64
        assert (page >= 0).all()
        for h in range(nh):
            g = h // (nh // nkv)
            keys = kp[page[:, None], g, ki[at]].double()               # [seen, hd]
            vals = vp[page[:, None], g, vi[at]].double()
            s = keys @ q[b, h * hd:(h + 1) * hd].double() / math.sqrt(hd)
            out[b, h * hd:(h + 1) * hd] = torch.softmax(s, 0) @ vals
    return out


def _case(seed, lens, nh, nkv, hd, window=0, sinks=0):
    """Random queries, a shuffled page table and filled pages for sequences of `lens` positions; with a
    window, pages that hold no visible position have been given back (-1 in the table)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    B, width = len(lens), (max(lens) + 63) // 64
    n_pages = B * width + 2
    perm = torch.randperm(n_pages, generator=g)[:B * width].reshape(B, width).to(torch.int32)
    table = torch.full((B, width), -1, dtype=torch.int32)
    for b, l in enumerate(lens):
        used = (l + 63) // 64
        table[b, :used] = perm[b, :used]
        for p in range(used):
            if window > 0 and not any(_visible(l - 1, t, window, sinks) for t in range(64 * p, 64 * p + 64)):
                table[b, p] = -1
    kp = torch.randn((n_pages, nkv, 64 * hd), generator=g).to(torch.bfloat16)
    vp = torch.randn((n_pages, nkv, 64 * hd), generator=g).to(torch.bfloat16)
    # queries four times as large as keys: scores spread over +-12, a few keys carry each head's weight, and a
    # page that is skipped or read twice moves the output by far more than rounding does
    q = (4 * torch.randn((B, nh * hd), generator=g)).to(torch.bfloat16)
    pos = torch.tensor([l - 1 for l in lens], dtype=torch.int32)
    return [t.to(DEV) for t in (q, kp, vp, table, pos)]


def _both(lib, lens, nh, nkv, hd, seed, window=0, sinks=0):
    q, kp, vp, table, pos = _case(seed, lens, nh, nkv, hd, window, sinks)
    B, width = table.shape
    scale = 1.0 / math.sqrt(hd)
    need = lib.llogos_attn_decode_workspace(B, nh, nkv, hd, width)
    assert 0 < need <= lib.llogos_attn_decode_static_capacity(), "the case must use the scratch array"
    ws = torch.empty(need, dtype=torch.float32, device=DEV)
    want = torch.zeros((B, nh * hd), dtype=torch.bfloat16, device=DEV)
    got = torch.zeros_like(want)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    torch.cuda.synchronize()
    code = lib.llogos_attn_decode_bf16(ptr(want), ptr(q), q.stride(0), ptr(kp), ptr(vp), ptr(table), width, width,
                                       ptr(pos), B, nh, nkv, hd, scale, window, sinks, ptr(ws), need, stream)
    assert code == 0, code
    code = lib.llogos_attn_decode_static_bf16(ptr(got), ptr(q), q.stride(0), ptr(kp), ptr(vp), ptr(table), width,
                                              width, ptr(pos), B, nh, nkv, hd, scale, window, sinks, stream)
    assert code == 0, code
    torch.cuda.synchronize()
    assert torch.isfinite(want.float()).all() and want.float().abs().max() > 0
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), \
        f"largest difference {(got.float() - want.float()).abs().max().item()}"
    plain = _plain(q, kp, vp, table, pos, nh, nkv, hd, window, sinks)
    err = (got.cpu().double() - plain).abs().max().item()
    assert err < 0.05, f"{err} from the plain attention (values of size 1, results rounded to bfloat16)"


def test_decode_attention_without_allocation_twice_in_a_row():
    lib = _lib()
    assert lib.llogos_attn_decode_static_init() == 0
    nh, nkv, hd = 8, 2, 128
    _both(lib, [1500, 70, 999, 64, 1, 1300], nh, nkv, hd, seed=1)      # 24 pages: six blocks along the context
    _both(lib, [700, 130, 65], nh, nkv, hd, seed=2)                    # smaller, over what the first call left
    _both(lib, [900, 5], 4, 4, 64, seed=3)                             # another head size and grouping
    _both(lib, [1500, 70, 999, 64, 1, 1300], nh, nkv, hd, seed=5)      # the array is full of a large call's results again
    # a window of 200 positions and 4 sinks: pages 1 to 19 of the longest sequence were given back, and the
    # blocks that would have read them write empty partial results over the stale ones
    _both(lib, [1490, 300, 66], nh, nkv, hd, seed=6, window=200, sinks=4)


def test_decode_attention_without_allocation_refuses_what_its_array_cannot_hold():
    lib = _lib()
    nh, nkv, hd = 32, 8, 128
    q, kp, vp, table, pos = _case(4, [100] * 64, nh, nkv, hd)
    width = 4096                                                       # as if the table were that wide
    assert lib.llogos_attn_decode_workspace(64, nh, nkv, hd, width) > lib.llogos_attn_decode_static_capacity()
    out = torch.zeros((64, nh * hd), dtype=torch.bfloat16, device=DEV)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    code = lib.llogos_attn_decode_static_bf16(ptr(out), ptr(q), q.stride(0), ptr(kp), ptr(vp), ptr(table),
                                              table.shape[1], width, ptr(pos), 64, nh, nkv, hd, 0.1, 0, 0,
                                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert code == -3
    torch.cuda.synchronize()
    assert not out.any()                                               # nothing was launched
