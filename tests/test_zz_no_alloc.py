"""The decode attention's entry point that allocates nothing (llogos_attn_decode_static_bf16),
called through ctypes as a caller outside the package would: its output must equal, bit for
bit, that of llogos_attn_decode_bf16 with a workspace from the caller, on two calls in a row
of which the second is smaller (the library's one scratch array keeps the first call's
contents), and a step that needs more scratch than the array holds must be refused."""
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


def _case(seed, lens, nh, nkv, hd):
    """Random queries, a shuffled page table and filled pages for sequences of `lens` positions."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    B, width = len(lens), (max(lens) + 63) // 64
    n_pages = B * width + 2
    perm = torch.randperm(n_pages, generator=g)[:B * width].reshape(B, width).to(torch.int32)
    table = torch.full((B, width), -1, dtype=torch.int32)
    for b, l in enumerate(lens):
        used = (l + 63) // 64
        table[b, :used] = perm[b, :used]
    kp = torch.randn((n_pages, nkv, 64 * hd), generator=g).to(torch.bfloat16)
    vp = torch.randn((n_pages, nkv, 64 * hd), generator=g).to(torch.bfloat16)
    q = torch.randn((B, nh * hd), generator=g).to(torch.bfloat16)
    pos = torch.tensor([l - 1 for l in lens], dtype=torch.int32)
    return [t.to(DEV) for t in (q, kp, vp, table, pos)]


def _both(lib, lens, nh, nkv, hd, seed):
    q, kp, vp, table, pos = _case(seed, lens, nh, nkv, hd)
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
                                       ptr(pos), B, nh, nkv, hd, scale, 0, 0, ptr(ws), need, stream)
    assert code == 0, code
    code = lib.llogos_attn_decode_static_bf16(ptr(got), ptr(q), q.stride(0), ptr(kp), ptr(vp), ptr(table), width,
                                              width, ptr(pos), B, nh, nkv, hd, scale, 0, 0, stream)
    assert code == 0, code
    torch.cuda.synchronize()
    assert torch.isfinite(want.float()).all() and want.float().abs().max() > 0
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), \
        f"largest difference {(got.float() - want.float()).abs().max().item()}"


def test_decode_attention_without_allocation_twice_in_a_row():
    lib = _lib()
    assert lib.llogos_attn_decode_static_init() == 0
    nh, nkv, hd = 8, 2, 128
    _both(lib, [1500, 70, 999, 64, 1, 1300], nh, nkv, hd, seed=1)      # 24 pages: six blocks along the context
    _both(lib, [700, 130, 65], nh, nkv, hd, seed=2)                    # smaller, over what the first call left
    _both(lib, [900, 5], 4, 4, 64, seed=3)                             # another head size and grouping


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
