"""Each kernel alone against a plain float64 / torch reference of the same op, at sizes
other than the engine's tests use (head sizes in steps of 16, widths and vocabularies that
are no power of two, many heads and groups)."""
import importlib
import math

import numpy as np
import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu
K = importlib.import_module("daisi-llogos_amd.ops.kernels")
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
RT = {"float32": 2e-6, "bfloat16": 1e-2}        # relative to the result's scale


def _t(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def _np(t):
    return t.detach().cpu().double().numpy()


def _close(got, want, dtype, scale=None):
    want = np.asarray(want, dtype=np.float64)
    scale = scale if scale is not None else max(1e-6, np.abs(want).max())
    err = np.abs(_np(got) - want).max() / scale
    assert err <= RT[dtype], f"relative error {err:.3e} > {RT[dtype]}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed(dtype):
    rng = np.random.default_rng(0)
    table = _t(rng.standard_normal((331, 200)), DT[dtype])
    ids = _t([0, 330, 7, 7, 129], torch.int32)
    out = K.embed(table, ids)
    assert out.dtype == torch.float32 and torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H", [80, 1000, 4100])
def test_rmsnorm(dtype, H):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((7, H)) * 3
    d = rng.standard_normal((7, H))
    w = 1 + 0.1 * rng.standard_normal(H)
    xd, dd, wd = _t(x), _t(d, DT[dtype]), _t(w)
    want = pm.rms_norm(x, w, 1e-5)
    _close(K.rmsnorm(xd, wd, 1e-5, DT[dtype]), want, dtype)
    # with a pending delta: the sum is written back in float32 and the norm is of the sum
    xs = x + _np(dd)
    out = K.rmsnorm(xd, wd, 1e-5, DT[dtype], delta=dd)
    assert np.abs(_np(xd) - xs).max() < 1e-6
    _close(out, pm.rms_norm(xs, w, 1e-5), dtype)
    # selected rows, no write back
    x2 = _t(x)
    rows = _t([6, 0, 3], torch.int32)
    out = K.rmsnorm(x2, wd, 1e-5, DT[dtype], delta=dd, rows=rows, write_back=False)
    assert torch.equal(x2, _t(x))
    _close(out, pm.rms_norm(xs[[6, 0, 3]], w, 1e-5), dtype)
    z = K.rmsnorm(torch.zeros(2, H, device=DEV), wd, 1e-6, DT[dtype])
    assert torch.count_nonzero(z) == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M,N,K_", [(1, 331, 80), (5, 96, 1000), (70, 130, 67), (200, 257, 129)])
def test_gemm(dtype, M, N, K_):
    rng = np.random.default_rng(2)
    a = _t(rng.standard_normal((M, K_)), DT[dtype])
    w = _t(rng.standard_normal((N, K_)) * 0.1, DT[dtype])
    b = _t(rng.standard_normal(N))
    want = pm.linear(_np(a), _np(w), _np(b))
    _close(K.gemm(a, w, b, DT[dtype]), want, dtype)
    _close(K.gemm(a, w, None, torch.float32), pm.linear(_np(a), _np(w)), "float32" if dtype == "float32" else dtype)
    # a view with a row stride (the first columns of a wider buffer) and the first rows of w
    wide = _t(rng.standard_normal((M, K_ + 13)), DT[dtype])
    _close(K.gemm(wide[:, :K_], w[:N // 2], None, DT[dtype]), pm.linear(_np(wide)[:, :K_], _np(w)[:N // 2]), dtype)
    # reference vector (tests/Daisi.Llogos.Tests/Cpu/MathOpsTests.cs:10-28)
    o = K.gemm(_t([[1, 2, 3], [4, 5, 6]], DT[dtype]), _t([[7, 9, 11], [8, 10, 12]], DT[dtype]), None, torch.float32)
    assert _np(o).tolist() == [[58, 64], [139, 154]]


@pytest.mark.parametrize("M,N,K_", [(1, 4096, 4096), (8, 331, 1000), (16, 100, 72), (17, 4096, 14336), (64, 257, 2048),
                                    (33, 6144, 4096), (5, 20000, 4096), (16, 70001, 1000), (7, 1000, 5120),
                                    (9, 333, 8192), (3, 200, 6000)])
def test_gemm_few_rows_on_the_matrix_cores(M, N, K_):
    rng = np.random.default_rng(7)
    a = _t(rng.standard_normal((M, K_)), torch.bfloat16)
    w = _t(rng.standard_normal((N, K_)) * 0.05, torch.bfloat16)
    b = _t(rng.standard_normal(N))
    want = pm.linear(_np(a), _np(w))
    scale = np.abs(want).max()
    for kernel, rbs in ((K.gemm_skinny_bf16, (1, 2, 4)), (K.gemm_skinny_lds_bf16, (1, 2))):
        for splits in (1, 2, 5, 8):
            for rb in rbs:
                out = kernel(a, w, None, torch.float32, splits, rb)
                assert out is not None and out.dtype == torch.float32 and out.shape[1:] == (M, N)
                assert np.abs(_np(out).sum(0) - want).max() <= 2e-6 * scale * math.sqrt(K_)
    if M <= 16 and K_ <= 8192:                                          # activations held in registers
        for strips in (1, 3, 8):
            out = K.gemm_skinny_stationary_bf16(a, w, b, torch.float32, strips)
            assert out is not None and np.abs(_np(out)[0] - (want + _np(b))).max() <= 2e-6 * scale * math.sqrt(K_)
    # silu(gate) * up made inside the product, from a bfloat16 row or from float32 partial sums
    if K_ % 16 == 0:
        I = K_ // 2
        act = pm.silu(_np(a)[:, :I]) * _np(a)[:, I:]
        act = _np(_t(act, torch.bfloat16))                              # the kernel rounds it to bfloat16
        want_sw = pm.linear(act, _np(w)[:, :I])
        w_half = w[:, :I].contiguous()
        for src in (a, torch.stack([a.float() * 0.25, a.float() * 0.75])):
            out = K.gemm_skinny_lds_bf16(src, w_half, None, torch.float32, 2, 1, swiglu=True)
            assert np.abs(_np(out).sum(0) - want_sw).max() <= 2e-2 * max(1.0, np.abs(want_sw).max())
    plain = K.gemm(a, w, b, torch.bfloat16)
    assert np.abs(_np(plain) - (want + _np(b))).max() <= 1e-2 * scale
    prod = K.gemm_product(a, w, torch.bfloat16)
    assert np.abs(_np(K.sum_parts(prod, b, torch.float32)) - (want + _np(b))).max() <= (1e-2 if prod.dtype == torch.bfloat16 else 1e-5) * scale
    # a row's result does not depend on how many other rows the batch has, bit for bit among
    # batches of up to 16, of 17 to 32 and of 33 to 64 rows (the plan is made for those classes),
    # and up to rounding between them
    if M > 1:
        fewest = 1 if M <= 16 else (17 if M <= 32 else 33)
        few = K.sum_parts(K.gemm_product(a[:fewest], w, torch.bfloat16), None, torch.float32)
        many = K.sum_parts(prod, None, torch.float32)
        assert torch.equal(few, many[:fewest])
        alone = K.sum_parts(K.gemm_product(a[:1], w, torch.bfloat16), None, torch.float32)
        assert np.abs(_np(alone) - _np(many[:1])).max() <= 1e-2 * scale
    assert K.gemm_skinny_bf16(a[:, :K_ - 4], w[:, :K_ - 4].contiguous(), None, torch.float32) is None   # k % 8


@pytest.mark.parametrize("M,N,K_", [(65, 257, 2048), (96, 4096, 14336), (97, 100, 1000), (128, 5120, 17408), (111, 333, 72)])
def test_gemm_of_65_to_128_rows_on_the_matrix_cores(M, N, K_):
    """The LDS few-row product at 65 to 128 rows: every number of blocks along k and both widths
    of a wave's strip of w; a row's result is the same bit for bit for every batch of this class."""
    rng = np.random.default_rng(8)
    a = _t(rng.standard_normal((M, K_)), torch.bfloat16)
    w = _t(rng.standard_normal((N, K_)) * 0.05, torch.bfloat16)
    b = _t(rng.standard_normal(N))
    want = pm.linear(_np(a), _np(w))
    scale = np.abs(want).max()
    for splits in (1, 3, 8):
        for rb in (1, 2):
            out = K.gemm_skinny_lds_bf16(a, w, None, torch.float32, splits, rb)
            assert out is not None and out.dtype == torch.float32 and out.shape[1:] == (M, N)
            assert np.abs(_np(out).sum(0) - want).max() <= 2e-6 * scale * math.sqrt(K_)
    out = K.gemm_skinny_lds_bf16(a, w, b, torch.bfloat16, 1, 1)
    assert np.abs(_np(out)[0] - (want + _np(b))).max() <= 1e-2 * scale
    assert K.gemm_skinny_lds_bf16(torch.cat([a, a]), w, None, torch.float32, 1, 1) is None            # more than 128 rows
    assert K.gemm_skinny_lds_bf16(a.float().repeat(1, 2), w, None, torch.float32, 1, 1, swiglu=True) is None  # fused producer: 64 rows
    prod = K.gemm_product(a, w, torch.bfloat16, f32_ok=True)
    assert (prod.dim() == 3) == (K.long_inner(w) and K.lds_splits(M, N, K_) > 1)
    many = K.sum_parts(prod, None, torch.float32)
    assert np.abs(_np(many) - want).max() <= (1e-5 if prod.dtype == torch.float32 else 1e-2) * scale
    if K.long_inner(w):
        few = K.sum_parts(K.gemm_product(a[:65], w, torch.bfloat16, f32_ok=True), None, torch.float32)
        assert torch.equal(few, many[:65])


@pytest.mark.parametrize("M,N,K_", [(17, 3000, 1024), (33, 16 * 9 * 5 + 7, 2048), (64, 4096, 4096), (100, 777, 512), (128, 2048, 640)])
def test_gemm_with_operands_straight_into_lds(M, N, K_):
    """The third form of the few-row product: every height of its blocks and several numbers
    of blocks along k; its results equal the LDS few-row product's bit for bit for the same
    parts of k, whatever the height."""
    rng = np.random.default_rng(9)
    a = _t(rng.standard_normal((M, K_)), torch.bfloat16)
    w = _t(rng.standard_normal((N, K_)) * 0.05, torch.bfloat16)
    b = _t(rng.standard_normal(N))
    want = pm.linear(_np(a), _np(w))
    scale = np.abs(want).max()
    for splits in (1, 2, 5):
        same = K.gemm_skinny_lds_bf16(a, w, None, torch.float32, splits, 1)
        for strips in (2, 3, 4, 7, 9):
            out = K.gemm_strips_bf16(a, w, None, torch.float32, splits, strips)
            assert out is not None and out.shape == same.shape
            assert np.abs(_np(out).sum(0) - want).max() <= 2e-6 * scale * math.sqrt(K_)
            assert torch.equal(out, same), (splits, strips)
    out = K.gemm_strips_bf16(a, w, b, torch.bfloat16, 1, 7)
    assert np.abs(_np(out)[0] - (want + _np(b))).max() <= 1e-2 * scale
    wide = _t(rng.standard_normal((M, K_ + 24)), torch.bfloat16)              # a view with a row stride
    out = K.gemm_strips_bf16(wide[:, :K_], w, None, torch.float32, 1, 8)
    assert np.abs(_np(out)[0] - pm.linear(_np(wide)[:, :K_], _np(w))).max() <= 2e-6 * scale * math.sqrt(K_)
    assert K.gemm_strips_bf16(a[:, :K_ - 8], w[:, :K_ - 8].contiguous(), None, torch.float32, 1, 7) is None   # k % 64
    assert K.gemm_strips_bf16(a, w, None, torch.float32, 1, 10) is None                                       # too high


def test_tall_products_through_the_dispatch_take_the_third_form():
    """A matrix as tall as the Qwen3-14B gate/up projection, few columns: the plan for 17 to 64
    rows is the third form, and a row's result is the same for every batch of such a class."""
    rng = np.random.default_rng(10)
    N, K_ = 34816, 1024
    w = torch.randn((N, K_), device=DEV, dtype=torch.bfloat16, generator=torch.Generator(device=DEV).manual_seed(3)) * 0.05
    a = _t(rng.standard_normal((64, K_)), torch.bfloat16)
    assert K.skinny_plan(33, N, K_)[0] == "strips" and K.skinny_plan(64, N, K_) == K.skinny_plan(33, N, K_)
    many = K.sum_parts(K.gemm_product(a, w, torch.bfloat16, f32_ok=True), None, torch.float32)
    few = K.sum_parts(K.gemm_product(a[:33], w, torch.bfloat16, f32_ok=True), None, torch.float32)
    assert torch.equal(few, many[:33])
    want = _np(a.float() @ w.float().t())
    assert np.abs(_np(many) - want).max() <= 2e-5 * max(1.0, np.abs(want).max())
    plain = K.gemm(a, w, None, torch.float32)
    assert np.abs(_np(plain) - want).max() <= 2e-5 * max(1.0, np.abs(want).max())


def test_products_of_random_shapes_through_the_dispatch():
    """Whatever kernel and split of k the plan picks for a shape, the product is right: row
    counts up to 64 and beyond, widths and depths that are multiples of 8 and of nothing else."""
    rng = np.random.default_rng(21)
    for case in range(40):
        M = int(rng.choice([1, 2, 5, 8, 13, 16, 17, 31, 33, 64, 70, 100, 128, 130]))
        K_ = 8 * int(rng.integers(1, 1100))                                # up to 8,792
        N = int(rng.integers(1, 40000)) if case % 4 else int(rng.integers(16384, 72000))
        if case % 5 == 3:
            N = int(rng.integers(1, K_ // 2 + 2))                           # few rows of w for its length
        a = _t(rng.standard_normal((M, K_)), torch.bfloat16)
        w = torch.randn((N, K_), device=DEV, dtype=torch.bfloat16, generator=torch.Generator(device=DEV).manual_seed(case)) * 0.05
        b = _t(rng.standard_normal(N))
        want = _np(a.float() @ w.float().t())                              # float32 on the device stands in for float64 here
        scale = max(1.0, np.abs(want).max())
        prod = K.gemm_product(a, w, torch.bfloat16, f32_ok=bool(case % 2))
        got = _np(K.sum_parts(prod, b, torch.float32))
        tol = (1e-2 if prod.dtype == torch.bfloat16 else 2e-5) * scale
        assert np.abs(got - (want + _np(b))).max() <= tol, (case, M, N, K_, K.skinny_plan(M, N, K_))
        got = _np(K.gemm(a, w, b, torch.float32))
        assert np.abs(got - (want + _np(b))).max() <= 2e-5 * scale, (case, M, N, K_)


def test_prompt_products_of_random_shapes_on_packed_weights():
    """Prompts through the dispatch with a packed copy at hand: whatever the plan picks (the tiled product in one
    part or in parts of k for matrices much longer than high, the library's elsewhere), every number of stages of
    64 and every way they fall into parts, heights below one block of rows, token counts that fill no tile."""
    rng = np.random.default_rng(33)
    seen = set()
    for case in range(36):
        M = int(rng.choice([129, 130, 190, 256, 257, 300, 511, 512, 513, 700, 1024]))
        K_ = 64 * int(rng.integers(1, 40)) if case % 3 else 64 * int(rng.choice([9, 10, 11, 13, 17, 18, 19, 35]))
        N = int(rng.integers(1, max(2, K_ // 2))) if case % 2 else int(rng.integers(1, 3000))
        a = _t(rng.standard_normal((M, K_)), torch.bfloat16)
        w = torch.randn((N, K_), device=DEV, dtype=torch.bfloat16, generator=torch.Generator(device=DEV).manual_seed(case)) * 0.05
        pw = K.pack_weights(w)
        want = _np(a.float() @ w.float().t())
        scale = max(1.0, np.abs(want).max())
        plan = K.tiles_plan(M, N, K_)
        seen.add(plan)
        prod = K.gemm_product(a, w, torch.bfloat16, f32_ok=True, packed=pw)
        assert (prod.dim() == 3 and prod.shape[0] == plan[0]) if plan is not None and plan[0] > 1 else prod.shape[-2:] == (M, N)
        got = _np(K.sum_parts(prod, None, torch.float32))
        assert np.abs(got - want).max() <= (1e-2 if prod.dtype == torch.bfloat16 else 2e-5) * scale, (case, M, N, K_, plan)
        for parts in (2, 4):                                               # every split the kernel takes, whether the plan asks for it or not
            if K_ // 64 // parts >= 2:
                got = K.gemm_tiles_bf16(a, pw, None, torch.float32, parts=parts, token_tiles=int(rng.choice([0, 2, 4])))
                assert got.shape == (parts, M, N)
                assert np.abs(_np(got.sum(0)) - want).max() <= 2e-5 * scale, (case, M, N, K_, parts)
    assert {p[0] for p in seen if p is not None} >= {1, 2, 4} and None in seen        # what the cases were drawn to cover


@pytest.mark.parametrize("N,K_", [(70, 16), (2048, 8192), (17000, 1000), (33000, 2049), (66000, 530), (5, 4099), (300, 7)])
def test_float32_product_of_few_rows_is_the_tiled_product_bit_for_bit(N, K_):
    """Up to 32 rows in float32 go to a kernel of their own (a wave a few columns, the rows of a in
    registers); it adds in the order of the tiled kernel, so a row's result is the same bits
    whichever of the two a step's row count selects, alone or beside others, and right."""
    rng = np.random.default_rng(N)
    a = _t(rng.standard_normal((40, K_)))
    w = _t(rng.standard_normal((N, K_)) * 0.05)
    b = _t(rng.standard_normal(N))
    tiled = K.gemm_generic(a, w, b, torch.float32)                         # 40 rows: the tiled kernel
    want = pm.linear(_np(a), _np(w), _np(b))
    assert np.abs(_np(tiled) - want).max() <= 2e-6 * max(1.0, np.abs(want).max()) * math.sqrt(K_)
    for M in (1, 2, 3, 4, 7, 8, 9, 16, 31, 32):
        few = K.gemm_generic(a[:M], w, b, torch.float32)
        assert torch.equal(few, tiled[:M]), (M, N, K_, (few - tiled[:M]).abs().max().item())
    # several tiles of rows: the same bits again
    big = torch.cat([a, _t(rng.standard_normal((160, K_)))])
    out = K.gemm_generic(big, w, b, torch.float32)
    assert torch.equal(out[:40], tiled)
    assert torch.equal(out[195:200], K.gemm_generic(big[195:200].contiguous(), w, b, torch.float32))
    wide = _t(rng.standard_normal((5, K_ + 3)))                            # rows that do not start at a multiple of 16 bytes
    few = K.gemm_generic(wide[:, :K_], w, None, torch.float32)
    many = K.gemm_generic(torch.cat([wide, wide * 0 + 1.0] * 4)[:, :K_], w, None, torch.float32)
    assert torch.equal(few, many[:5])


def test_rope_table_is_double_precision():
    pos = _t([0, 1, 4095, 100000], torch.int32)
    f = pm.rope_frequencies(64, 5e5)
    cs = _np(K.rope_table(pos, _t(f, torch.float64)))
    ang = np.array([0, 1, 4095, 100000])[:, None] * f[None, :]
    assert np.abs(cs[..., 0] - np.cos(ang)).max() < 1e-7 and np.abs(cs[..., 1] - np.sin(ang)).max() < 1e-7


def _page_index(hd):
    """(keys, values): index tensors [64, hd] of where (token, dimension) lies in one kv head's part
    of a page, by the cache's own rule (cache/pages.py)."""
    pages = importlib.import_module("daisi-llogos_amd.cache.pages")
    ki, vi = pages.page_offsets(hd)
    return torch.tensor(ki, device=DEV), torch.tensor(vi, device=DEV)


def _pages(n_seqs, max_len, rng):
    """A shuffled page table: sequences' pages lie anywhere in the pool."""
    per = (max_len + 63) // 64
    ids = rng.permutation(n_seqs * per + 3)[:n_seqs * per].reshape(n_seqs, per)
    return ids.astype(np.int32), n_seqs * per + 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd,rot,pairing,norm", [
    (4, 2, 16, 16, 0, False), (6, 1, 32, 32, 0, True), (5, 5, 48, 24, 0, True), (8, 2, 80, 80, 1, False),
    (3, 3, 128, 64, 1, True), (2, 1, 256, 256, 0, False), (8, 2, 128, 128, 0, True), (5, 5, 128, 128, 0, False)])
@pytest.mark.parametrize("lens,new", [([70, 3], [5, 3]), ([70, 30], [40, 27])])
def test_qk_rope_cache(dtype, nh, nkv, hd, rot, pairing, norm, lens, new):
    """Two sequences; this step brings the last `new` tokens of each: a few tokens, and runs
    that cross a page's end and start in the middle of one."""
    rng = np.random.default_rng(3)
    T = sum(new)
    tok_seq = np.repeat(np.arange(2), new).astype(np.int32)
    tok_pos = np.concatenate([np.arange(l - n, l) for l, n in zip(lens, new)]).astype(np.int32)
    table, n_pages = _pages(2, 70, rng)
    width = (nh + 2 * nkv) * hd
    qkv = _t(rng.standard_normal((T, width)), DT[dtype])
    bias = _t(rng.standard_normal(width)) if norm else None              # bias and norm together: bias first
    orig = _np(qkv) + (_np(bias) if bias is not None else 0)
    qw = 1 + 0.1 * rng.standard_normal(hd)
    kw = 1 + 0.1 * rng.standard_normal(hd)
    f = pm.rope_frequencies(rot, 1e4)
    cs = K.rope_table(_t(tok_pos, torch.int32), _t(f, torch.float64))
    kp = torch.zeros((n_pages, nkv, 64 * hd), dtype=DT[dtype], device=DEV)
    vp = torch.zeros((n_pages, nkv, 64 * hd), dtype=DT[dtype], device=DEV)
    args = (nh, nkv, hd, rot, pairing, _t(qw) if norm else None, _t(kw) if norm else None, 1e-5,
            cs, kp, vp, _t(table, torch.int32), _t(tok_seq, torch.int32), _t(tok_pos, torch.int32))
    q_out = K.qk_rope_cache(qkv, bias, DT[dtype], *args)
    # the same projection as three float32 partial sums gives the same result
    third = qkv.float() / 4
    q_parts = K.qk_rope_cache(torch.stack([third, 2 * third, third]), bias, DT[dtype], *args)
    assert torch.equal(q_parts, q_out)
    q, k, v = orig[:, :nh * hd], orig[:, nh * hd:(nh + nkv) * hd], orig[:, (nh + nkv) * hd:]
    if norm:
        q = pm.per_head_rms_norm(q, qw, nh, hd, 1e-5)
        k = pm.per_head_rms_norm(k, kw, nkv, hd, 1e-5)
    rope = pm.rope_split_half if pairing == 0 else pm.rope_interleaved
    q, k = rope(q, tok_pos, nh, hd, f), rope(k, tok_pos, nkv, hd, f)
    _close(q_out, q, dtype)
    kc, vc = _np(kp), _np(vp)
    ki, vi = (_np(i).astype(np.int64) for i in _page_index(hd))
    for t in range(T):
        page = table[tok_seq[t], tok_pos[t] // 64]
        got_k = kc[page][:, ki[tok_pos[t] % 64]].reshape(-1)
        got_v = vc[page][:, vi[tok_pos[t] % 64]].reshape(-1)
        assert np.abs(got_k - k[t]).max() <= RT[dtype] * max(1, np.abs(k).max())
        assert np.abs(got_v - v[t]).max() <= RT[dtype] * max(1, np.abs(v).max())
    assert np.count_nonzero(kc) == T * nkv * hd and np.count_nonzero(vc) == T * nkv * hd   # nothing else was written


def _attention_case(dtype, nh, nkv, hd, lens, new, window=0, sinks=0, seed=4, scale_q=1.0):
    """Fills a paged cache with random keys and values for sequences of `lens` positions, of
    which the last `new` are this step's queries; returns the kernel's and the plain result."""
    rng = np.random.default_rng(seed)
    B, T = len(lens), sum(new)
    table, n_pages = _pages(B, max(lens), rng)
    kp = torch.zeros((n_pages, nkv, 64 * hd), dtype=DT[dtype], device=DEV)
    vp = torch.zeros((n_pages, nkv, 64 * hd), dtype=DT[dtype], device=DEV)
    ki, vi = _page_index(hd)
    ks = [rng.standard_normal((l, nkv * hd)) for l in lens]
    vs = [rng.standard_normal((l, nkv * hd)) for l in lens]
    for b in range(B):
        kb, vb = _t(ks[b], DT[dtype]), _t(vs[b], DT[dtype])
        ks[b], vs[b] = _np(kb), _np(vb)
        for p0 in range(0, lens[b], 64):                                # page by page
            n = min(64, lens[b] - p0)
            kp[table[b, p0 // 64]][:, ki[:n]] = kb[p0:p0 + n].view(n, nkv, hd).permute(1, 0, 2)
            vp[table[b, p0 // 64]][:, vi[:n]] = vb[p0:p0 + n].view(n, nkv, hd).permute(1, 0, 2)
    stride = nh * hd + 24                                               # queries sit in a wider row
    qbuf = _t(rng.standard_normal((T, stride)) * scale_q, DT[dtype])
    tok_seq = np.repeat(np.arange(B), new).astype(np.int32)
    tok_pos = np.concatenate([np.arange(l - n, l) for l, n in zip(lens, new)]).astype(np.int32)
    return dict(q=qbuf, stride=stride, kp=kp, vp=vp, ki=ki, vi=vi, table=_t(table, torch.int32), ks=ks, vs=vs,
                tok_seq=tok_seq, tok_pos=tok_pos, new=new, lens=lens)


def _plain_attention(c, nh, nkv, hd, window=0, sinks=0, scale=None):
    outs = []
    q = _np(c["q"])[:, :nh * hd]
    o = 0
    for b, (l, n) in enumerate(zip(c["lens"], c["new"])):
        full_q = np.zeros((l, nh * hd))
        full_q[l - n:] = q[o:o + n]
        outs.append(pm.attention(full_q, c["ks"][b], c["vs"][b], nh, nkv, hd, scale=scale, window=window,
                                 sinks=sinks, rows=range(l - n, l))[l - n:])
        o += n
    return np.concatenate(outs)


ATTN_SHAPES = [(4, 2, 16), (6, 1, 32), (5, 5, 48), (8, 2, 64), (6, 3, 80), (4, 1, 96), (7, 7, 112),
               (32, 8, 128), (3, 1, 256)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd", ATTN_SHAPES)
def test_attention_whole_prompts_and_single_tokens(dtype, nh, nkv, hd):
    for lens, new in (([70, 3, 130], [70, 3, 130]),                     # whole prompts
                      ([300, 1, 65, 64], [1, 1, 1, 1]),                 # one token each
                      ([200, 90], [72, 5])):                            # continued prompts
        c = _attention_case(dtype, nh, nkv, hd, lens, new)
        ctx = type("Ctx", (), dict(tok_seq=_t(c["tok_seq"], torch.int32), tok_pos=_t(c["tok_pos"], torch.int32),
                                   is_decode=max(new) == 1, max_context=max(lens), batch=len(lens),
                                   n_tokens=sum(new), cu_seqlens=np.concatenate([[0], np.cumsum(new)]).tolist(),
                                   cu_dev=_t(np.concatenate([[0], np.cumsum(new)]), torch.int32),
                                   starts=[l - n for l, n in zip(lens, new)], shared={}))()
        out = K.attention(ctx, c["q"], c["stride"], c["kp"], c["vp"], c["table"], nh, nkv, hd, 1 / math.sqrt(hd))
        _close(out, _plain_attention(c, nh, nkv, hd), dtype)


@pytest.mark.parametrize("window,sinks", [(0, 0), (200, 70)])
@pytest.mark.parametrize("nh,nkv,hd,batch,longest", [(8, 4, 128, 64, 700),      # one block a sequence, three pages a wave
                                                     (8, 4, 64, 70, 1500),       # batches beyond the captured sizes
                                                     (16, 2, 64, 128, 700),
                                                     (8, 4, 128, 4, 1500),       # one page a wave, six blocks merged
                                                     (4, 1, 128, 4, 3300),       # 13 blocks merged
                                                     (8, 2, 128, 16, 5000)])     # several pages a wave and several blocks
def test_single_token_attention_with_blocks_of_every_size(nh, nkv, hd, batch, longest, window, sinks):
    """The decode kernel gives a wave more pages when there are many blocks; every form must
    agree with the plain attention, whatever the lengths of the other sequences.  With a window
    the pages between the sinks and the window are not the sequence's any more (the cache gives
    them back): they hold NaN here, which would spoil the result if a wave took one of them."""
    rng = np.random.default_rng(batch)
    lens = [int(x) for x in rng.integers(1, longest // 3, batch)]
    lens[1], lens[batch // 2], lens[-1] = longest, 64, 65
    new = [1] * batch
    c = _attention_case("bfloat16", nh, nkv, hd, lens, new, seed=batch)
    for b, l in enumerate(lens):                                        # unwritten page tails must not matter
        if l % 64:
            page = int(c["table"][b, l // 64])
            c["kp"][page][:, c["ki"][l % 64:]] = float("nan")
            c["vp"][page][:, c["vi"][l % 64:]] = float("nan")
        for pi in range((l + 63) // 64 if window else 0):
            if pi * 64 >= sinks and pi * 64 + 63 <= l - 1 - window:     # no key of the page is visible from position l - 1
                page = int(c["table"][b, pi])
                c["kp"][page] = float("nan")
                c["vp"][page] = float("nan")
    ctx = type("Ctx", (), dict(tok_seq=_t(c["tok_seq"], torch.int32), tok_pos=_t(c["tok_pos"], torch.int32),
                               is_decode=True, max_context=max(lens), batch=batch, n_tokens=batch,
                               cu_seqlens=list(range(batch + 1)), cu_dev=None, starts=[l - 1 for l in lens],
                               shared={}))()
    out = K.attention_mfma_bf16(ctx, c["q"], c["stride"], c["kp"], c["vp"], c["table"], nh, nkv, hd, 1 / math.sqrt(hd),
                                window, sinks)
    assert out is not None
    _close(out, _plain_attention(c, nh, nkv, hd, window, sinks), "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_of_random_shapes(dtype):
    """Heads, groups, head sizes, lengths, windows and sinks drawn at random: prompts whole and
    continued, and single tokens, whichever kernel the dispatch takes."""
    rng = np.random.default_rng(31)
    for case in range(24):
        hd = int(rng.choice([16, 32, 48, 64, 64, 96, 128, 128, 256]))
        nkv = int(rng.choice([1, 2, 3, 8]))
        nh = nkv * int(rng.choice([1, 2, 4, 5, 16]))
        B = int(rng.integers(1, 5))
        lens = [int(rng.integers(1, 400)) for _ in range(B)]
        kind = case % 3
        new = [1] * B if kind == 0 else (lens if kind == 1 else [int(rng.integers(1, l + 1)) for l in lens])
        window = int(rng.choice([0, 0, 1, 64, 100]))
        sinks = int(rng.choice([0, 4])) if window else 0
        c = _attention_case(dtype, nh, nkv, hd, lens, new, seed=100 + case)
        for b, l in enumerate(lens):                                        # unwritten page tails must not matter
            if l % 64:
                page = int(c["table"][b, l // 64])
                c["kp"][page][:, c["ki"][l % 64:]] = float("nan")
                c["vp"][page][:, c["vi"][l % 64:]] = float("nan")
        ctx = type("Ctx", (), dict(tok_seq=_t(c["tok_seq"], torch.int32), tok_pos=_t(c["tok_pos"], torch.int32),
                                   is_decode=max(new) == 1, max_context=max(lens), batch=B, n_tokens=sum(new),
                                   cu_seqlens=np.concatenate([[0], np.cumsum(new)]).tolist(),
                                   cu_dev=_t(np.concatenate([[0], np.cumsum(new)]), torch.int32),
                                   starts=[l - n for l, n in zip(lens, new)], shared={}))()
        out = K.attention(ctx, c["q"], c["stride"], c["kp"], c["vp"], c["table"], nh, nkv, hd, 1 / math.sqrt(hd), window, sinks)
        want = _plain_attention(c, nh, nkv, hd, window, sinks)
        err = np.abs(_np(out) - want).max()
        assert err <= RT[dtype] * max(1.0, np.abs(want).max()), (case, nh, nkv, hd, lens, new, window, sinks, err)


@pytest.mark.parametrize("tile_rows,halves", [(64, 1), (128, 1), (128, 2)])
@pytest.mark.parametrize("nh,nkv,hd", [(6, 2, 64), (8, 2, 128), (3, 3, 128)])
@pytest.mark.parametrize("window,sinks", [(0, 0), (100, 0), (70, 5)])
def test_prompt_attention_on_the_matrix_cores(tile_rows, halves, nh, nkv, hd, window, sinks):
    """The prompt kernels (pages read by each wave; pages shared through LDS by one set of waves
    or by two that take the pages in turn) on long and short sequences, whole and continued,
    with pages half written, and with odd and even numbers of pages a tile."""
    K.PREFILL_TILE_ROWS, K.PREFILL_HALVES = tile_rows, halves
    try:
        for lens, new in (([300, 129, 5, 64], [300, 129, 5, 64]), ([400, 90, 257], [200, 33, 129]),
                          ([1100, 700], [1100, 190])):
            c = _attention_case("bfloat16", nh, nkv, hd, lens, new, seed=11)
            ctx = type("Ctx", (), dict(tok_seq=_t(c["tok_seq"], torch.int32), tok_pos=_t(c["tok_pos"], torch.int32),
                                       is_decode=False, max_context=max(lens), batch=len(lens), n_tokens=sum(new),
                                       cu_seqlens=np.concatenate([[0], np.cumsum(new)]).tolist(),
                                       cu_dev=_t(np.concatenate([[0], np.cumsum(new)]), torch.int32),
                                       starts=[l - n for l, n in zip(lens, new)], shared={}))()
            # what lies behind the written part of a page must not matter: poison it
            for b, l in enumerate(lens):
                if l % 64:
                    page = int(c["table"][b, l // 64])
                    c["kp"][page][:, c["ki"][l % 64:]] = float("nan")
                    c["vp"][page][:, c["vi"][l % 64:]] = float("nan")
            out = K.attention_mfma_bf16(ctx, c["q"], c["stride"], c["kp"], c["vp"], c["table"], nh, nkv, hd,
                                        1 / math.sqrt(hd), window, sinks)
            assert out is not None
            _close(out, _plain_attention(c, nh, nkv, hd, window, sinks), "bfloat16")
    finally:
        K.PREFILL_TILE_ROWS = K.PREFILL_HALVES = 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_finds_a_far_key_among_hundreds(dtype):
    """One early key matches the query strongly; the output must be its value."""
    nh, nkv, hd, L = 4, 2, 64, 700
    c = _attention_case(dtype, nh, nkv, hd, [L], [1], scale_q=0.01)
    q = c["q"]
    far = 5
    page, off = int(c["table"][0, far // 64]), far % 64
    key = torch.zeros(hd, device=DEV); key[3] = 40.0
    c["kp"][page][:, c["ki"][off]] = key.to(c["kp"].dtype)
    q[0, :nh * hd] = (key.repeat(nh) * 2).to(q.dtype)                   # score 40 * 80 / 8 = 400 for that key
    ctx = type("Ctx", (), dict(tok_seq=_t(c["tok_seq"], torch.int32), tok_pos=_t(c["tok_pos"], torch.int32),
                               is_decode=True, max_context=L, batch=1, n_tokens=1, cu_seqlens=[0, 1], cu_dev=None,
                               starts=[L - 1], shared={}))()
    out = _np(K.attention(ctx, q, c["stride"], c["kp"], c["vp"], c["table"], nh, nkv, hd, 1 / math.sqrt(hd)))
    want = np.concatenate([c["vs"][0][far].reshape(nkv, hd)[h // 2] for h in range(nh)])
    assert np.abs(out[0] - want).max() < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hd", [32, 64, 128])
@pytest.mark.parametrize("window,sinks", [(64, 0), (70, 0), (5, 2), (128, 64), (1, 0)])
def test_attention_window_edges(dtype, window, sinks, hd):
    nh, nkv = 4, 2
    for lens, new in (([300, 66], [1, 1]), ([200, 10], [200, 10]), ([257], [100])):
        c = _attention_case(dtype, nh, nkv, hd, lens, new, seed=9)
        # keys just outside and just inside the window stand out, so an off-by-one shows
        for b, l in enumerate(lens):
            for p in (l - 1 - window, l - window):
                if p >= max(sinks, 0) and p >= 0:
                    page, off = int(c["table"][b, p // 64]), p % 64
                    c["kp"][page][:, c["ki"][off]] *= 6.0
                    c["ks"][b][p] = _np(c["kp"][page][:, c["ki"][off]]).reshape(-1)    # as stored
        ctx = type("Ctx", (), dict(tok_seq=_t(c["tok_seq"], torch.int32), tok_pos=_t(c["tok_pos"], torch.int32),
                                   is_decode=max(new) == 1, max_context=max(lens), batch=len(lens),
                                   n_tokens=sum(new), cu_seqlens=np.concatenate([[0], np.cumsum(new)]).tolist(),
                                   cu_dev=_t(np.concatenate([[0], np.cumsum(new)]), torch.int32),
                                   starts=[l - n for l, n in zip(lens, new)], shared={}))()
        out = K.attention(ctx, c["q"], c["stride"], c["kp"], c["vp"], c["table"], nh, nkv, hd, 1 / math.sqrt(hd),
                          window, sinks)
        _close(out, _plain_attention(c, nh, nkv, hd, window, sinks), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_swiglu(dtype):
    rng = np.random.default_rng(5)
    gu = _t(rng.standard_normal((9, 2 * 137)) * 4, DT[dtype])
    g, u = _np(gu)[:, :137], _np(gu)[:, 137:]
    _close(K.swiglu(gu), pm.silu(g) * u, dtype)
    parts = torch.stack([gu.float() * 0.25, gu.float() * 0.75])
    _close(K.swiglu(parts, DT[dtype]), pm.silu(g) * u, dtype)
    _close(K.sum_parts(parts, None, DT[dtype]), _np(gu), dtype)


def test_gather_of_token_ids():
    src = _t([5, 9, 2, 7, 11], torch.int32)
    rows = _t([4, 0, 0, 3], torch.int32)
    dst = torch.full((4,), -1, dtype=torch.int32, device=DEV)
    K.gather_i32(dst, src, rows)
    assert dst.cpu().tolist() == [11, 5, 5, 7]
    K.gather_i32(dst, src, _t([1, 7, -1, 2], torch.int32))               # rows outside the vector give 0, never a fault
    assert dst.cpu().tolist() == [9, 0, 0, 2]
    with pytest.raises(K.KernelError):
        K.gather_i32(dst, src, rows[:3])
    with pytest.raises(K.KernelError):
        K.gather_i32(dst, src.float(), rows)


def test_argmax_first_maximum_wins():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((5, 128257)).astype(np.float32)
    x[1, 4000] = x[1, 90000] = 9.0                                      # a tie: the first wins
    x[2, 128256] = 10.0
    x[3, :] = 0.25                                                      # all equal
    x[4, 0] = 11.0
    got = K.argmax(_t(x)).cpu().tolist()
    assert got == [int(np.argmax(x[0])), 4000, 128256, 0, 0]
    assert K.argmax(_t([[1., 5., 3., 2.]])).item() == 1                 # tests/.../SamplerTests.cs:8-18


def test_kernels_refuse_what_they_cannot_do():
    x = torch.zeros(4, 64, device=DEV)
    with pytest.raises(K.KernelError, match="GPU"):
        K.rmsnorm(torch.zeros(4, 64), torch.ones(64), 1e-6, torch.float32)
    with pytest.raises(K.KernelError, match="weight"):
        K.rmsnorm(x, torch.ones(63, device=DEV), 1e-6, torch.float32)
    with pytest.raises(K.KernelError, match="w must be"):
        K.gemm(x, torch.zeros(8, 65, device=DEV), None, torch.float32)
    with pytest.raises(K.KernelError, match="not supported"):
        K.gemm(x.half(), torch.zeros(8, 64, device=DEV).half(), None, torch.float16)
    with pytest.raises(K.KernelError, match="head_dim"):
        K.qk_rope_cache(torch.zeros(1, 3 * 1024, device=DEV), None, torch.float32, 1, 1, 1024, 2, 0, None, None, 1e-6,
                        torch.zeros(1, 1, 2, device=DEV), None, None, None,
                        torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("M,N,K_", [(1, 4096, 4096), (8, 331, 1000), (16, 100, 72), (17, 4096, 14336), (33, 257, 2048),
                                    (64, 1000, 520), (48, 6144, 4096), (5, 64, 32), (64, 65, 8)])
def test_gemm_on_packed_weights(M, N, K_):
    """The few-row product on the packed copy of the weights (blocks of 64 rows, steps of 32 k,
    zero-padded): every row count class, heights and lengths that fill no block or step, one part
    and several, bias, float32 and bfloat16 results."""
    rng = np.random.default_rng(M * 1000 + N)
    a, w = _t(rng.standard_normal((M, K_)), torch.bfloat16), _t(rng.standard_normal((N, K_)) * 0.05, torch.bfloat16)
    bias = _t(rng.standard_normal(N))
    want = _np(a) @ _np(w).T
    pw = K.pack_weights(w)
    assert pw.N == N and pw.K == K_ and pw.data.numel() == -(-N // 64) * 64 * -(-K_ // 32) * 32
    for chunk in (128, 256):
        for splits in (1, 2, 5):
            out = K.gemm_packed_bf16(a, pw, None, torch.float32, splits, chunk)
            assert out is not None and out.dtype == torch.float32
            _close(out.sum(0), want, "float32", scale=np.abs(want).max() * 10)        # bfloat16 operands, float32 sums
        out = K.gemm_packed_bf16(a, pw, bias, torch.bfloat16, 1, chunk)
        _close(out[0], want + _np(bias), "bfloat16")
    # through the dispatch, as a part calls it
    out = K.gemm_product(a, w, torch.bfloat16, f32_ok=True, packed=pw)
    _close(K.sum_parts(out, None, torch.float32), want, "float32", scale=np.abs(want).max() * 10)
    _close(K.gemm(a, w, bias, torch.float32, packed=pw), want + _np(bias), "float32", scale=np.abs(want).max() * 10)
    # a row's result does not depend on the other rows of its class
    if M > 1:
        alone = K.gemm_packed_bf16(a[:1].contiguous(), pw, None, torch.float32, 1, 256)
        if (M + 15) // 16 in (1,):
            assert torch.equal(alone[0], K.gemm_packed_bf16(a, pw, None, torch.float32, 1, 256)[0][:1])


def test_first_rows_of_packed_weights_and_the_fused_swiglu():
    rng = np.random.default_rng(3)
    I, H = 200, 136
    w = _t(rng.standard_normal((192, H)) * 0.1, torch.bfloat16)
    pw = K.pack_weights(w)
    a = _t(rng.standard_normal((9, H)), torch.bfloat16)
    first = pw.rows(128)
    assert first is not None and first.N == 128 and pw.rows(100) is None and pw.rows(192) is pw
    _close(K.gemm_packed_bf16(a, first, None, torch.float32, 1, 128)[0], (_np(a) @ _np(w).T)[:, :128], "float32", scale=50.0)
    # down product of silu(gate) * up made on the way, from a bfloat16 row [gate | up] and from float32 partial sums
    wd = _t(rng.standard_normal((H, I)) * 0.1, torch.bfloat16)
    pd = K.pack_weights(wd)
    gu = _t(rng.standard_normal((9, 2 * I)), torch.bfloat16)
    g, u = _np(gu)[:, :I], _np(gu)[:, I:]
    act = _np(_t(pm.silu(g) * u, torch.bfloat16))                     # the kernel rounds the product to bfloat16
    want = act @ _np(wd).T
    out = K.gemm_packed_bf16(gu, pd, None, torch.float32, 1, 128, swiglu=True)
    _close(out[0], want, "bfloat16")
    parts = _t(rng.standard_normal((3, 9, 2 * I)))
    tot = _np(parts).sum(0)
    want = _np(_t(pm.silu(tot[:, :I]) * tot[:, I:], torch.bfloat16)) @ _np(wd).T
    out = K.gemm_packed_bf16(parts, pd, None, torch.float32, 2, 128, swiglu=True)
    _close(out.sum(0), want, "bfloat16")


@pytest.mark.parametrize("M,I,H", [(1, 208, 136), (9, 14336, 4096), (16, 64, 72), (33, 1008, 264), (64, 2048, 520), (47, 16, 40)])
def test_gate_up_product_with_the_swiglu_epilogue(M, I, H):
    """The few-row product on a matrix packed as strips of gate rows and up rows in turn gives
    silu(a gate^T) * (a up^T) directly; against the plain functions, every class of row count,
    widths that fill no block."""
    rng = np.random.default_rng(M + I)
    wg, wu = (_t(rng.standard_normal((I, H)) * 0.08, torch.bfloat16) for _ in range(2))
    a = _t(rng.standard_normal((M, H)), torch.bfloat16)
    w = torch.cat([wg, wu]).contiguous()
    pw = K.pack_weights(w, gate_rows=I)
    assert pw.gate_rows == I and pw.rows(64) is None
    want = pm.silu(_np(a) @ _np(wg).T) * (_np(a) @ _np(wu).T)
    for chunk in (128, 256):
        got = K.gemm_packed_gated_bf16(a, pw, torch.float32, chunk)
        assert got is not None and got.shape == (M, I)
        _close(got, want, "float32", scale=np.abs(want).max() * 50)           # hardware exp2 and reciprocal: about 1e-6 relative
    _close(K.gemm_packed_gated_bf16(a, pw, torch.bfloat16, 256), want, "bfloat16")
    # a packed copy in this order serves no other product: the dispatch leaves it aside
    out = K.gemm_product(a, w, torch.bfloat16, packed=pw)
    _close(K.sum_parts(out, None, torch.float32), _np(a) @ _np(w).T, "bfloat16")
    with pytest.raises(K.KernelError):
        K.pack_weights(w, gate_rows=I + 16)


@pytest.mark.parametrize("M,N,K_", [(1, 4096, 4096), (8, 4096, 14336), (16, 48, 200), (5, 80, 8), (13, 5120, 1000), (3, 16, 72), (9, 120, 200),
                                    (2, 7, 16)])
@pytest.mark.parametrize("waves,strips", [(4, 1), (8, 1), (16, 1), (8, 2), (4, 2)])
def test_product_that_adds_itself_to_the_residual_stream(M, N, K_, waves, strips):
    """x += a w^T + bias in one kernel for up to 16 rows, with what it leaves for the norm that follows: the
    sums of squares of the new rows by strips of 16 columns, and x * norm_w rounded to bfloat16.  Against
    float64; rows beyond M stay zero in the sums; a row's result does not depend on the rows beside it."""
    rng = np.random.default_rng(M * 100 + N + waves + strips)
    a, w = _t(rng.standard_normal((M, K_)), torch.bfloat16), _t(rng.standard_normal((N, K_)) * 0.05, torch.bfloat16)
    bias, norm_w = _t(rng.standard_normal(N)), _t(1 + 0.1 * rng.standard_normal(N))
    x0 = _t(rng.standard_normal((M, N)) * 3)
    pw = K.pack_weights(w)
    want = _np(x0) + _np(a) @ _np(w).T + _np(bias)
    x = x0.clone()
    left = K.gemm_residual_bf16(x, a, pw, bias, waves, norm_w, strips)
    assert isinstance(left, K.RowSquares) and left.width == N and left.norm_w is norm_w
    _close(x, want, "float32", scale=np.abs(want).max() * 10)                    # bfloat16 operands, float32 sums
    n_strips = -(-(-(-N // 16)) // strips)                                        # blocks of 16 * strips columns
    assert left.sums.shape == (n_strips, 16)
    sums = _np(left.sums)
    assert np.all(sums[:, M:] == 0)
    padded = np.zeros((M, n_strips * 16 * strips))
    padded[:, :N] = _np(x)
    by_strip = (padded ** 2).reshape(M, n_strips, 16 * strips).sum(2).T                      # [strips, M] of the x it wrote
    assert np.allclose(sums[:, :M], by_strip, rtol=2e-6, atol=1e-30)
    assert torch.equal(left.unscaled, (x * norm_w).to(torch.bfloat16))           # the same float32 product, rounded once
    # without a bias and without the norm's rows; one row alone gives the same bits
    x1 = x0.clone()
    plain = K.gemm_residual_bf16(x1, a, pw, None, waves, strips=strips)
    assert plain.unscaled is None
    _close(x1, want - _np(bias), "float32", scale=np.abs(want).max() * 10)
    alone = x0[:1].clone()
    K.gemm_residual_bf16(alone, a[:1].contiguous(), pw, None, waves, strips=strips)
    assert torch.equal(alone, x1[:1])
    # refused: more than 16 rows, a packed gate/up matrix
    assert K.gemm_residual_bf16(torch.zeros(17, N, device=DEV), torch.zeros(17, K_, device=DEV, dtype=torch.bfloat16), pw, None, waves) is None


def test_library_product_that_adds_itself_to_the_residual_stream():
    """For prompts that the library's product serves, the sum with the residual stream is the product's
    epilogue: the float32 product added to x, bit for bit; refused for few rows, other element types and where
    the tiled product serves."""
    rng = np.random.default_rng(5)
    for M, N, K_ in ((200, 96, 72), (2048, 4096, 4096), (129, 331, 1000)):
        a, w = _t(rng.standard_normal((M, K_)), torch.bfloat16), _t(rng.standard_normal((N, K_)) * 0.05, torch.bfloat16)
        x0 = _t(rng.standard_normal((M, N)) * 3)
        x = x0.clone()
        assert K.gemm_library_add(x, a, w)
        assert torch.equal(x, x0 + torch.mm(a, w.t(), out_dtype=torch.float32))
        _close(x, _np(x0) + _np(a) @ _np(w).T, "float32", scale=np.abs(_np(x)).max() * 10)
    x = x0[:64].clone()
    assert not K.gemm_library_add(x, a[:64].contiguous(), w) and torch.equal(x, x0[:64])
    assert not K.gemm_library_add(x0.clone(), a.float(), w.float())
    a, w = _t(rng.standard_normal((256, 8192)), torch.bfloat16), _t(rng.standard_normal((1024, 8192)) * 0.05, torch.bfloat16)
    pw = K.pack_weights(w)
    if K.tiles_plan(256, 1024, 8192) is not None:                              # much longer than high: the tiled product in parts
        assert not K.gemm_library_add(torch.zeros(256, 1024, device=DEV), a, w, pw)


@pytest.mark.parametrize("M,N,K_", [(1, 6144, 4096), (8, 331, 1000), (16, 96, 72), (7, 64, 4112), (11, 200, 16)])
def test_product_on_norm_rows_without_their_scale(M, N, K_):
    """The few-row product whose activations are x * w of an rmsnorm, with the sums of squares of x beside
    them: the row's scale 1 / sqrt(mean square + eps) is applied to the result.  Against float64 on the same
    bfloat16 rows; parts and a bias; any number of partial sums (also more than 256 and fewer than 16)."""
    rng = np.random.default_rng(M + N)
    eps = 1e-5
    x = _t(rng.standard_normal((M, K_)) * 2)
    norm_w = _t(1 + 0.1 * rng.standard_normal(K_))
    w = _t(rng.standard_normal((N, K_)) * 0.05, torch.bfloat16)
    bias = _t(rng.standard_normal(N))
    pw = K.pack_weights(w)
    unscaled = (x * norm_w).to(torch.bfloat16)
    inv = 1.0 / np.sqrt((_np(x) ** 2).mean(1) + eps)
    want = (_np(unscaled) @ _np(w).T) * inv[:, None]
    for strips in (K_ // 8, 3, 300):                                               # the sums arrive in parts of any count
        cols = np.array_split(np.arange(K_), strips)
        sums = np.zeros((strips, 16))
        for i, c in enumerate(cols):
            sums[i, :M] = (_np(x)[:, c] ** 2).sum(1)
        left = K.RowSquares(_t(sums), K_, unscaled, norm_w)
        for splits, chunk in ((1, 128), (3, 256)):
            out = K.gemm_packed_unscaled_bf16(left, eps, pw, None, torch.float32, splits, chunk)
            assert out is not None and out.dtype == torch.float32
            _close(out.sum(0), want, "float32", scale=np.abs(want).max() * 10)
        out = K.gemm_packed_unscaled_bf16(left, eps, pw, bias, torch.bfloat16, 1, 128)
        _close(out[0], want + _np(bias), "bfloat16")
    # the norm's own kernel and the product on its output: the same up to one rounding of the activations
    normed = K.rmsnorm(x.clone(), norm_w, eps, torch.bfloat16)
    ref = K.gemm_packed_bf16(normed, pw, None, torch.float32, 1, 128)[0]
    _close(K.gemm_packed_unscaled_bf16(left, eps, pw, None, torch.float32, 1, 128)[0], _np(ref), "bfloat16")


@pytest.mark.parametrize("M,I,H", [(1, 208, 136), (8, 14336, 4096), (16, 64, 72)])
def test_gate_up_product_on_norm_rows_without_their_scale(M, I, H):
    rng = np.random.default_rng(M + I)
    eps = 1e-6
    wg, wu = (_t(rng.standard_normal((I, H)) * 0.08, torch.bfloat16) for _ in range(2))
    pw = K.pack_weights(torch.cat([wg, wu]).contiguous(), gate_rows=I)
    x = _t(rng.standard_normal((M, H)) * 4)
    norm_w = _t(1 + 0.1 * rng.standard_normal(H))
    unscaled = (x * norm_w).to(torch.bfloat16)
    strips = -(-H // 16)
    sums = np.zeros((strips, 16))
    for i in range(strips):
        sums[i, :M] = (_np(x)[:, 16 * i: 16 * i + 16] ** 2).sum(1)
    inv = 1.0 / np.sqrt((_np(x) ** 2).mean(1) + eps)
    a = _np(unscaled)
    want = pm.silu((a @ _np(wg).T) * inv[:, None]) * ((a @ _np(wu).T) * inv[:, None])
    left = K.RowSquares(_t(sums), H, unscaled, norm_w)
    for chunk in (128, 256):
        got = K.gemm_packed_unscaled_bf16(left, eps, pw, None, torch.float32, 1, chunk)
        assert got is not None and got.shape == (M, I)
        _close(got, want, "float32", scale=np.abs(want).max() * 50)
    _close(K.gemm_packed_unscaled_bf16(left, eps, pw, None, torch.bfloat16, 1, 128), want, "bfloat16")


@pytest.mark.parametrize("M,N,K_", [(65, 256, 64), (300, 1000, 512), (2048, 4096, 4096), (129, 6144, 1024), (700, 130, 192),
                                    (1500, 2300, 640), (190, 136, 576), (318, 40, 576)])
@pytest.mark.parametrize("token_tiles", [0, 4, 2])
def test_tiled_product_for_many_rows_on_packed_weights(M, N, K_, token_tiles):
    """The hand-written prompt-size product (tiles of 256 or 128 tokens x 256 rows, 32x32x16 MFMAs on the
    packed copy): token counts and heights that fill no tile, float32 and bfloat16 results, bias, parts of k."""
    rng = np.random.default_rng(M + N)
    a, w = _t(rng.standard_normal((M, K_)), torch.bfloat16), _t(rng.standard_normal((N, K_)) * 0.05, torch.bfloat16)
    bias = _t(rng.standard_normal(N))
    want = _np(a) @ _np(w).T
    pw = K.pack_weights(w)
    _close(K.gemm_tiles_bf16(a, pw, None, torch.float32, token_tiles=token_tiles), want, "float32", scale=np.abs(want).max() * 10)
    _close(K.gemm_tiles_bf16(a, pw, bias, torch.bfloat16, token_tiles=token_tiles), want + _np(bias), "bfloat16")
    assert K.gemm_tiles_bf16(a[:, :K_ - 8].contiguous(), K.pack_weights(w[:, :K_ - 8].contiguous()), None, torch.float32) is None
    for parts in (2, 3, 4):                                             # (9 stages in 4 parts: 2, 2, 2 and 3, none empty)
        got = K.gemm_tiles_bf16(a, pw, None, torch.bfloat16, parts=parts, token_tiles=token_tiles)
        if K_ // 64 // parts < 2:
            assert got is None                                          # a part would hold less than two stages of 64
            continue
        assert got.shape == (parts, M, N) and got.dtype == torch.float32
        if parts == 2:                                                  # the first part is the product over the first half of k
            half = (K_ // 64) // 2 * 64
            _close(got[0], _np(a)[:, :half] @ _np(w)[:, :half].T, "float32", scale=np.abs(want).max() * 10)
        _close(got.sum(0), want, "float32", scale=np.abs(want).max() * 10)
        _close(K.sum_parts(got, bias, torch.float32), want + _np(bias), "float32", scale=np.abs(want).max() * 10)


def test_tiled_product_cuts_the_last_round_into_smaller_tiles():
    """2,048 tokens by 7,168 rows are 8 x 28 tiles of 256 tokens: on 64 compute units 224 tiles are three
    rounds and a half, and the launch takes the row tiles of the half round in tiles of 128 tokens.  The
    result does not depend on the cut (every element's sum runs over k in the same order)."""
    rng = np.random.default_rng(3)
    M, N, K_ = 2048, 7168, 256
    a, w = _t(rng.standard_normal((M, K_)), torch.bfloat16), _t(rng.standard_normal((N, K_)) * 0.05, torch.bfloat16)
    pw = K.pack_weights(w)
    lib = K._lib()
    outs = []
    for units in (64, 256, 1):                    # 224 tiles: 3.5 rounds of 64 (cut), less than one round of 256, whole rounds of 1
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
        code = lib.llogos_gemm_tiles_bf16(K._p(out), K.F32, K._p(a), a.stride(0), K._p(pw.data), None, M, N, K_, N, M * N, 0, 1, 0,
                                          units, K._stream())
        assert code == 0
        outs.append(out)
    _close(outs[0], _np(a) @ _np(w).T, "float32", scale=np.abs(_np(a) @ _np(w).T).max() * 10)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


@pytest.mark.parametrize("M,I,H", [(200, 1008, 256), (2048, 14336, 4096), (65, 16, 64), (1000, 7200, 320)])
def test_tiled_product_with_the_swiglu_epilogue(M, I, H):
    rng = np.random.default_rng(M + I)
    wg, wu = (_t(rng.standard_normal((I, H)) * 0.08, torch.bfloat16) for _ in range(2))
    a = _t(rng.standard_normal((M, H)) * (0.25 if H > 1000 else 1.0), torch.bfloat16)
    pw = K.pack_weights(torch.cat([wg, wu]).contiguous(), gate_rows=I)
    want = pm.silu(_np(a) @ _np(wg).T) * (_np(a) @ _np(wu).T)
    for token_tiles in (0, 4, 2):
        got = K.gemm_tiles_bf16(a, pw, None, torch.float32, token_tiles=token_tiles)
        assert got.shape == (M, I)
        _close(got, want, "float32", scale=np.abs(want).max() * 50)
        _close(K.gemm_tiles_bf16(a, pw, None, torch.bfloat16, token_tiles=token_tiles), want, "bfloat16")
    with pytest.raises(K.KernelError):
        K.gemm_tiles_bf16(a, pw, None, torch.float32, parts=2)


def test_prompts_through_the_tiled_product(monkeypatch):
    """An engine whose prompt products are the hand-written ones gives the plain logits like the default."""
    import gpu_helpers as H
    monkeypatch.setattr(K, "PROMPT_PRODUCT", "tiles")
    name = "layer_8b"
    eng = H.engine(name, "bfloat16", max_tokens=64 * 8, n_slots=2)
    assert eng.model.layers[0].ffn.gate_up.packed.gate_rows == 14336
    toks = H.tokens(name, 150, 1)
    s = eng.alloc_slot()
    got = eng.step([(s, toks)], want="all").cpu().double().numpy()
    H.close(got, H.plain_logits(name, toks), "bfloat16", "prompt through the tiled product", config=name)


def test_long_prompts_take_the_tiled_gate_up_product_by_default():
    """From TILES_MIN_ROWS tokens on the gate/up product with its SwiGLU epilogue is the hand-written one;
    the logits are the plain ones either way, and the two ways agree within bfloat16 rounding."""
    import gpu_helpers as H
    assert K.PROMPT_PRODUCT == "auto" and K.tiles_serve_gated(K.TILES_MIN_ROWS, 4096) and not K.tiles_serve_gated(K.TILES_MIN_ROWS - 1, 4096)
    name = "layer_8b"
    eng = H.engine(name, "bfloat16", max_tokens=64 * 18, n_slots=1)
    toks = H.tokens(name, K.TILES_MIN_ROWS + 40, 2)
    calls = []
    real = K.gemm_tiles_bf16
    K.gemm_tiles_bf16 = lambda *a, **kw: (calls.append((a[0].shape[0], a[1].gate_rows > 0)), real(*a, **kw))[1]
    try:
        s = eng.alloc_slot()
        got = eng.step([(s, toks)], want=[[0, 100, len(toks) - 1]]).cpu().double().numpy()
    finally:
        K.gemm_tiles_bf16 = real
    assert calls == [(len(toks), True)] * 2                                # the gate/up product of both layers
    want = H.plain_logits(name, toks)[[0, 100, len(toks) - 1]]
    H.close(got, want, "bfloat16", "long prompt, tiled gate/up product", config=name)
