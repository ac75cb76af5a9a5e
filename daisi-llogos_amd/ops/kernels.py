"""Python face of the HIP kernels: argument checks, then one call into the library.

Every function checks on the host that shapes, element types and devices match what the
kernel and its grid assume, and raises before anything is launched.  Tensors are torch
tensors used as device memory; launches go to torch's current stream.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
import os
from typing import Optional, Sequence, Tuple

import torch

from . import library
from ..cache.pages import HEAD_DIM_STEP, MAX_HEAD_DIM, PAGE_TOKENS      # the one definition; the library is checked against PAGE_TOKENS when loaded

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}
MAX_BANNED = 64             # ids one sampling call can set to -inf (kMaxBanned in csrc/sampling.hip)


class KernelError(RuntimeError):
    """A kernel refused its arguments or failed to launch."""


def _lib():
    return library.load()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """torch's current stream of the current device, as the library takes it.  (The raw getter
    spares the ten microseconds a Stream object costs, once per launch.)"""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch._C._cuda_getDevice()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"element type {t.dtype} is not supported (float32 or bfloat16)") from None


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*tensors) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel arguments must live on the GPU")
            _need(t.is_contiguous(), "kernel arguments must be contiguous")


def _check(code: int, name: str) -> None:
    if code != 0:
        if code == -1:
            raise KernelError(f"{name}: bad argument")
        if code == -2:
            raise KernelError(f"{name}: size not supported")
        if code == -3:
            raise KernelError(f"{name}: larger than the library's fixed scratch array holds")
        raise KernelError(f"{name}: HIP error {code}")


def _i32(t: Optional[torch.Tensor], name: str) -> None:
    if t is not None:
        _need(t.dtype == torch.int32, f"{name} must be int32")


def _parts(t: Optional[torch.Tensor]) -> Tuple[int, int]:
    """(number of parts, elements between parts) of a product: [T, N] is one part,
    [P, T, N] are P partial sums that the consumer adds."""
    if t is None or t.dim() == 2:
        return 1, 0
    _need(t.dim() == 3, "a product must be [T, N] or [parts, T, N]")
    return t.shape[0], t.stride(0)


def _check_pools(k_pool: torch.Tensor, v_pool: torch.Tensor, n_kv_heads: int, head_dim: int, who: str) -> None:
    _need(head_dim % 16 == 0, f"{who}: head size {head_dim} is not a multiple of 16")
    _need(tuple(k_pool.shape[1:]) == (n_kv_heads, PAGE_TOKENS * head_dim),
          f"{who}: key pool must be [pages, kv_heads, {PAGE_TOKENS} * head_dim]")
    _need(tuple(v_pool.shape) == tuple(k_pool.shape),
          f"{who}: value pool must be [pages, kv_heads, {PAGE_TOKENS} * head_dim] like the key pool")
    _need(k_pool.is_contiguous() and v_pool.is_contiguous(), f"{who}: the pools must be contiguous")


# ----------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """float32 rows of `table` ([V, H], float32 or bfloat16) at int32 `ids`, times `scale`."""
    _dev(table, ids)
    _i32(ids, "ids")
    _need(table.dim() == 2 and ids.dim() == 1, "embed: table [V, H], ids [T]")
    T, H = ids.numel(), table.shape[1]
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _check(_lib().llogos_embed(_p(out), _p(table), _dt(table), _p(ids), T, H, ctypes.c_float(scale), _stream()), "embed")
    return out


def scale_softcap(x: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
    """In place on float32 `x`: x * scale, then with cap > 0 bent to cap * tanh(x / cap)."""
    _dev(x)
    _need(x.dtype == torch.float32 and cap >= 0, "scale_softcap: float32 values, cap >= 0")
    if x.numel():
        _check(_lib().llogos_scale_softcap(_p(x), ctypes.c_longlong(x.numel()), ctypes.c_float(scale),
                                           ctypes.c_float(cap), _stream()), "scale_softcap")
    return x


def gather_i32(dst: torch.Tensor, src: torch.Tensor, rows: torch.Tensor) -> None:
    """dst[i] = src[rows[i]] for int32 vectors on the device."""
    _dev(dst, src, rows)
    _i32(dst, "dst"); _i32(src, "src"); _i32(rows, "rows")
    _need(dst.dim() == 1 and src.dim() == 1 and rows.dim() == 1 and dst.numel() == rows.numel()
          and dst.is_contiguous() and src.is_contiguous() and rows.is_contiguous(), "gather_i32: contiguous vectors, dst like rows")
    _check(_lib().llogos_gather_i32(_p(dst), _p(src), _p(rows), dst.numel(), src.numel(), _stream()), "gather_i32")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
            write_back: bool = True) -> torch.Tensor:
    """RMSNorm of the float32 residual stream `x` [T, H] with the pending `delta` ([T, H] or
    partial sums [parts, T, H]) added first (and written back to `x` when `write_back`).
    With `rows` only those rows are normed, into a compact output."""
    _dev(x, weight, delta, rows)
    _i32(rows, "rows")
    _need(x.dtype == torch.float32 and x.dim() == 2, "rmsnorm: x must be float32 [T, H]")
    T, H = x.shape
    _need(weight.dtype == torch.float32 and weight.shape == (H,), "rmsnorm: weight must be float32 [H]")
    parts, part_stride = _parts(delta)
    if delta is not None:
        _need(tuple(delta.shape[-2:]) == tuple(x.shape), "rmsnorm: delta must have x's shape")
    R = rows.numel() if rows is not None else T
    out = torch.empty((R, H), dtype=out_dtype, device=x.device)
    if R == 0:
        return out
    _check(_lib().llogos_rmsnorm(_p(out), _DT[out_dtype], _p(x), _p(delta), _dt(delta) if delta is not None else F32,
                                 parts, ctypes.c_longlong(part_stride),
                                 _p(rows), _p(weight), ctypes.c_float(eps), R, H, int(write_back), _stream()),
           "rmsnorm")
    return out


def residual_add(x: torch.Tensor, delta: torch.Tensor) -> None:
    _dev(x, delta)
    _need(x.dtype == torch.float32 and delta.shape == x.shape, "residual_add: x float32, same shapes")
    _check(_lib().llogos_residual_add(_p(x), _p(delta), _dt(delta), ctypes.c_longlong(x.numel()), _stream()),
           "residual_add")


def gemm_generic(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [M, K] . w [N, K]^T (+ bias) with plain 32-bit FMAs."""
    _dev(w, bias)
    _need(a.is_cuda and a.dim() == 2 and a.stride(1) == 1, "gemm: a must be [M, K] with unit inner stride")
    M, K = a.shape
    _need(w.dim() == 2 and w.shape[1] == K, f"gemm: w must be [N, {K}], got {tuple(w.shape)}")
    N = w.shape[0]
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    else:
        _need(out.shape == (M, N) and out.dtype == out_dtype and out.stride(1) == 1, "gemm: bad out")
    if M == 0:
        return out
    _check(_lib().llogos_gemm_generic(_p(out), _dt(out), _p(a), _dt(a), _p(w), _dt(w), _p(bias),
                                      M, N, K, a.stride(0), out.stride(0), _stream()), "gemm_generic")
    return out


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """[T, half, 2] float32 (cos, sin) of positions[t] * inv_freq[i], computed in double."""
    _dev(positions, inv_freq)
    _i32(positions, "positions")
    _need(inv_freq.dtype == torch.float64 and inv_freq.dim() == 1, "rope_table: inv_freq must be float64 [half]")
    T, half = positions.numel(), inv_freq.numel()
    cs = torch.empty((T, half, 2), dtype=torch.float32, device=positions.device)
    _check(_lib().llogos_rope_table(_p(cs), _p(positions), _p(inv_freq), T, half, _stream()), "rope_table")
    return cs


def qk_rope_cache(qkv: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                  n_heads: int, n_kv_heads: int, head_dim: int, rot: int, pairing: int,
                  q_norm_w: Optional[torch.Tensor], k_norm_w: Optional[torch.Tensor], eps: float,
                  cs: torch.Tensor, k_pool: Optional[torch.Tensor], v_pool: Optional[torch.Tensor],
                  table: Optional[torch.Tensor], tok_seq: torch.Tensor, tok_pos: torch.Tensor) -> torch.Tensor:
    """From the fused projection rows [q | k | v] ([T, W] or partial sums [parts, T, W], plus
    `bias` [W]): per-head norm (optional) and rotation of q and k; q is returned
    [T, n_heads * head_dim] in `out_dtype`, k and v go to their cache pages."""
    _dev(qkv, bias, q_norm_w, k_norm_w, cs, k_pool, v_pool, table, tok_seq, tok_pos)
    _i32(tok_seq, "tok_seq"); _i32(tok_pos, "tok_pos"); _i32(table, "table")
    parts, part_stride = _parts(qkv)
    T = qkv.shape[-2]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    _need(qkv.shape[-1] == width, f"qk_rope_cache: qkv must be [T, {width}]")
    _need(qkv.dtype == out_dtype or qkv.dtype == torch.float32, "qk_rope_cache: qkv must be float32 or the cache's type")
    _need(0 < head_dim <= MAX_HEAD_DIM, f"qk_rope_cache: head_dim {head_dim} not in 1..{MAX_HEAD_DIM}")
    _need(rot % 2 == 0 and 0 <= rot <= head_dim, "qk_rope_cache: rotary dimension must be even and <= head_dim")
    _need(cs.dtype == torch.float32 and cs.shape == (T, rot // 2, 2), "qk_rope_cache: rotary table shape")
    _need(tok_seq.numel() == T and tok_pos.numel() == T, "qk_rope_cache: per-token arrays must have T entries")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (width,), f"qk_rope_cache: bias must be float32 [{width}]")
    for wgt in (q_norm_w, k_norm_w):
        if wgt is not None:
            _need(wgt.dtype == torch.float32 and wgt.shape == (head_dim,), "qk_rope_cache: norm weight float32 [head_dim]")
    if n_kv_heads > 0:
        _need(k_pool is not None and v_pool is not None and table is not None, "qk_rope_cache: cache missing")
        _need(k_pool.dtype == out_dtype and v_pool.dtype == out_dtype, "qk_rope_cache: cache type differs")
        _check_pools(k_pool, v_pool, n_kv_heads, head_dim, "qk_rope_cache")
        _need(table.dim() == 2, "qk_rope_cache: page table must be [batch, pages]")
    q_out = torch.empty((T, n_heads * head_dim), dtype=out_dtype, device=qkv.device)
    _check(_lib().llogos_qk_rope_cache(
        _p(qkv), _dt(qkv), parts, ctypes.c_longlong(part_stride), qkv.stride(-2), _p(bias), _p(q_out), _DT[out_dtype],
        n_heads, n_kv_heads, head_dim, rot, pairing,
        _p(q_norm_w), _p(k_norm_w), ctypes.c_float(eps), _p(cs), _p(k_pool), _p(v_pool),
        _p(table), table.stride(0) if table is not None else 0, _p(tok_seq), _p(tok_pos), T, _stream()),
        "qk_rope_cache")
    return q_out


def attention_generic(q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                      table: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor,
                      n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                      window: int = 0, sinks: int = 0) -> torch.Tensor:
    """Attention of T query rows (row stride `q_stride` elements, heads first) over the
    paged cache; returns [T, n_heads * head_dim] in the cache's element type."""
    _dev(k_pool, v_pool, table, tok_seq, tok_pos)
    _i32(tok_seq, "tok_seq"); _i32(tok_pos, "tok_pos"); _i32(table, "table")
    T = tok_seq.numel()
    _need(q.is_cuda and q.dtype == k_pool.dtype, "attention: q and cache types differ")
    _need(n_heads % n_kv_heads == 0, "attention: heads must be a multiple of kv heads")
    _need(0 < head_dim <= MAX_HEAD_DIM, f"attention: head_dim {head_dim} not in 1..{MAX_HEAD_DIM}")
    _check_pools(k_pool, v_pool, n_kv_heads, head_dim, "attention")
    _need(q_stride >= n_heads * head_dim and q.numel() >= (T - 1) * q_stride + n_heads * head_dim,
          "attention: q too small")
    out = torch.empty((T, n_heads * head_dim), dtype=q.dtype, device=q.device)
    _check(_lib().llogos_attention_generic(
        _p(out), _p(q), _dt(q), q_stride, _p(k_pool), _p(v_pool), _p(table), table.stride(0),
        _p(tok_seq), _p(tok_pos), T, n_heads, n_kv_heads, head_dim, ctypes.c_float(scale),
        window, sinks, _stream()), "attention_generic")
    return out


def swiglu(gu: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """silu(gate) * up from fused rows [gate | up] ([T, 2 I] or partial sums [parts, T, 2 I])."""
    _dev(gu)
    parts, part_stride = _parts(gu)
    _need(gu.shape[-1] % 2 == 0, "swiglu: rows must be [gate | up]")
    out_dtype = out_dtype or gu.dtype
    _need(gu.dtype == out_dtype or gu.dtype == torch.float32, "swiglu: input must be float32 or the output's type")
    T, I = gu.shape[-2], gu.shape[-1] // 2
    out = torch.empty((T, I), dtype=out_dtype, device=gu.device)
    _check(_lib().llogos_swiglu(_p(out), _DT[out_dtype], _p(gu), _dt(gu), parts, ctypes.c_longlong(part_stride),
                                T, I, _stream()), "swiglu")
    return out


def sum_parts(product: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype) -> torch.Tensor:
    """One plain [T, N] tensor of `out_dtype` from a product that may come in parts, plus bias."""
    _dev(product, bias)
    parts, part_stride = _parts(product)
    if parts == 1 and bias is None and product.dtype == out_dtype:
        return product if product.dim() == 2 else product[0]
    _need(parts == 1 or product.dtype == torch.float32, "sum_parts: parts must be float32")
    T, N = product.shape[-2:]
    out = torch.empty((T, N), dtype=out_dtype, device=product.device)
    _check(_lib().llogos_sum_parts(_p(out), _DT[out_dtype], _p(product), _dt(product), parts, ctypes.c_longlong(part_stride),
                                   _p(bias), T, N, _stream()), "sum_parts")
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """int32 index of the first maximum of each row of float32 logits."""
    _dev(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "argmax: logits must be float32 [R, V]")
    R, V = logits.shape
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _check(_lib().llogos_argmax(_p(out), _p(logits), R, V, _stream()), "argmax")
    return out


# ----------------------------------------------------------------------------
# dispatch: which kernel serves a call
# ----------------------------------------------------------------------------
_compute_units = {}


def compute_units(device=None) -> int:
    """Compute units of the GPU the products are planned for, read from the device once (256 on
    an MI355X; that number also stands in where no GPU is visible, for planning on the host)."""
    if not torch.cuda.is_available():
        return 256
    index = torch.cuda.current_device() if device is None else torch.device(device).index or 0
    if index not in _compute_units:
        _compute_units[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return _compute_units[index]


SKINNY_MAX_ROWS = 64
LDS_MAX_ROWS = 128          # rows the LDS few-row product takes without a fused producer


def lds_splits(M: int, N: int, K: int, n_cus: Optional[int] = None) -> int:
    """Blocks along k for the LDS few-row product.  Measured on the MI355X, three things decide:
    how evenly the blocks fill the compute units (544 blocks on 256 units run as long as 768),
    whether there are enough of them to keep the memory system busy (about 1.5 a unit), and the
    float32 partial sums every further block along k writes and the consumer reads (they cost
    about 6 M / K of the weights' time each).  64 and more rows of activations leave LDS for two
    blocks a unit, so blocks come in rounds of twice the units there.  More blocks along k are taken only
    for a clear gain (8 %), since they also cost the consumer a fused form or a launch."""
    n_cus = n_cus or compute_units()
    n_blocks = -(-N // 64)
    chunks = -(-K // 256)
    rows = 16 if M <= 16 else (32 if M <= 32 else (64 if M <= 64 else 128))
    per_round = n_cus * (2 if rows >= 64 else 1)
    best, best_score, seen = 1, -1.0, set()
    for s in range(1, 9):
        per = -(-chunks // s)
        parts = -(-chunks // per)
        if parts in seen or (parts > 1 and per < 2):
            continue
        seen.add(parts)
        blocks = n_blocks * parts
        evenness = blocks / (-(-blocks // per_round) * per_round)
        enough = min(1.0, blocks / (1.5 * n_cus))
        partial_sums = 1.0 + (parts - 1) * 6.0 * rows / K
        score = evenness * enough / partial_sums * (1.0 - 0.01 * (parts - 1))
        if score > best_score * 1.08:
            best, best_score = parts, score
    return best


def stationary_strips(N: int, K: int, n_cus: Optional[int] = None) -> int:
    """Strips of 16 rows of w a block of the activation-stationary product streams.  More strips
    spread the activations' loads over more weights; the blocks must still fill the compute
    units evenly (598 blocks on 256 units were measured at 3.9 TB/s where 448 reach 5.5) and
    leave about seven waves a unit."""
    n_cus = n_cus or compute_units()
    waves = 4 if K <= 4096 else 8
    n_strips = -(-N // 16)
    best, best_score = 2, -1.0
    for strips in range(2, 17):
        blocks = -(-n_strips // strips)
        evenness = blocks / (-(-blocks // n_cus) * n_cus)
        enough = min(1.0, blocks * waves / (7.0 * n_cus))
        score = evenness * enough / (1.0 + 0.4 / strips)
        if score >= best_score:
            best, best_score = strips, score
    return best


def resident_strips(M: int, N: int, K: int, n_cus: Optional[int] = None) -> Optional[Tuple[int, int]]:
    """(parts of k, strips per block) for the few-row product whose operands go straight into
    LDS, or None where it is not the faster one.  It pays for 17 to 64 rows on a tall, large
    matrix when its blocks, 5 to 9 strips high, are all resident at once (two to a compute
    unit) and fill most of those places, while the LDS few-row product's 64-row blocks either
    need a second round or leave a fifth more of the places empty: then the activations are
    read once per 80 to 144 rows of w and nothing waits for a second round (measured on the
    gate/up matrices of eight model sizes: 6 to 20 % faster where this says so, level or
    slower where it does not, among them everything below 24576 rows)."""
    if not (16 < M <= 64 and N >= 24576 and K % 64 == 0):
        return None
    n_cus = n_cus or compute_units()
    places = 2 * n_cus
    other = -(-N // 64) * lds_splits(M, N, K, n_cus)
    other_fill = other / places if other <= places else 0.0
    n_strips = -(-N // 16)
    best, best_fill = None, 0.0
    for strips in (9, 8, 7, 6, 5):
        for parts in (1, 2):
            if parts > 1 and K < 512 * parts:
                continue
            blocks = -(-n_strips // strips) * parts
            if blocks <= places and blocks / places > best_fill:
                best, best_fill = (parts, strips), blocks / places
    if best is None or best_fill < 0.75 or best_fill - other_fill < 0.2:
        return None
    return best


def skinny_plan(M: int, N: int, K: int) -> Tuple[str, int, int]:
    """(kernel, blocks along k, 16-row blocks of w per wave) for the few-row product.
    'strips': both operands straight into LDS, blocks of several strips (see resident_strips).
    'stationary': activations held in registers while strips of w stream past; best for few
    rows and very many rows of w (gate/up, the head).  'regs': every wave fetches its own
    activation fragments; for up to 4 rows where k is too long for 'stationary'.  'lds': the
    block shares the activations through LDS; its speed hardly depends on the number of rows.
    The plan depends on the shape and on the number of rows rounded up to 16, 32 or 64, so a
    row's additions come in the same order for every batch of that class."""
    if N >= 16384 and K <= 4096 and (M <= 8 or (M <= 16 and N >= 65536)):
        return "stationary", 1, stationary_strips(N, K)       # third value: strips per block
    if N >= 16384 and 4096 < K <= 8192 and M <= 16:           # 8 waves a block
        return "stationary", 1, stationary_strips(N, K)
    if M <= 4 and N >= 16384:
        strips = -(-N // 16)
        return "regs", max(1, min(-(-1024 // strips), K // 1024, 8)), 1
    resident = resident_strips(M, N, K)
    if resident is not None:
        return "strips", resident[0], resident[1]             # third value: strips per block
    return "lds", lds_splits(M, N, K), 1


def long_inner(w: torch.Tensor) -> bool:
    """Whether w [N, K] has few rows for its length (a feed-forward's down projection).  For 65
    to 128 rows of activations the library's product leaves most compute units idle on such a
    matrix (75 us measured for [4096, 14336] at 128 rows, 1.6 TB/s), and the LDS few-row
    product with blocks along k is faster (44 us); on the other layer shapes the library is."""
    return w.dtype == torch.bfloat16 and w.shape[1] >= 2 * w.shape[0]


def gemm_skinny_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                     splits: int = 1, row_blocks: int = 1) -> Optional[torch.Tensor]:
    """The few-row bfloat16 product on the matrix cores: [parts, M, N], where parts > 1 are
    float32 partial sums over ranges of k that the consumer adds (then no bias is applied
    here).  None when the shape is not one the kernel takes."""
    M, K = a.shape
    N = w.shape[0]
    if not (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and 0 < M <= SKINNY_MAX_ROWS and K % 8 == 0
            and a.stride(1) == 1 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and w.is_contiguous()):
        return None
    _dev(w, bias)
    _need(w.dim() == 2 and w.shape[1] == K, f"gemm: w must be [N, {K}], got {tuple(w.shape)}")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    lib = _lib()
    parts = lib.llogos_gemm_skinny_parts(K, int(splits))
    if parts > 1:
        _need(bias is None, "gemm: a product in parts leaves the bias to its consumer")
        out_dtype = torch.float32
    out = torch.empty((parts, M, N), dtype=out_dtype, device=a.device)
    code = lib.llogos_gemm_skinny_bf16(
        _p(out), _DT[out_dtype], _p(a), _p(w), _p(bias), M, N, K, a.stride(0), N,
        ctypes.c_longlong(M * N), int(splits), int(row_blocks), _stream())
    if code == -2:
        return None
    _check(code, "gemm_skinny_bf16")
    return out


def gemm_skinny_stationary_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor],
                                out_dtype: torch.dtype, strips: int = 4) -> Optional[torch.Tensor]:
    """The few-row bfloat16 product with the activations held in registers while `strips` strips
    of 16 rows of w stream past: up to 16 rows, K <= 8192.  [1, M, N]; None for other shapes."""
    if a.dim() != 2:
        return None
    M, K = a.shape
    N = w.shape[0]
    if not (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and 0 < M <= 16 and K <= 8192 and K % 8 == 0
            and a.stride(1) == 1 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and w.is_contiguous()):
        return None
    _dev(w, bias)
    _need(w.dim() == 2 and w.shape[1] == K, f"gemm: w must be [N, {K}], got {tuple(w.shape)}")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    out = torch.empty((1, M, N), dtype=out_dtype, device=a.device)
    code = _lib().llogos_gemm_skinny_stationary_bf16(
        _p(out), _DT[out_dtype], _p(a), _p(w), _p(bias), M, N, K, a.stride(0), N, int(strips), _stream())
    if code == -2:
        return None
    _check(code, "gemm_skinny_stationary_bf16")
    return out


def gemm_skinny_lds_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                         splits: int = 1, row_blocks: int = 1, swiglu: bool = False) -> Optional[torch.Tensor]:
    """The few-row bfloat16 product with the activations shared through LDS: [parts, M, N].
    With `swiglu`, `a` is the fused gate/up product ([M, 2 K] bfloat16 or float32 partial sums
    [parts, M, 2 K]) and silu(gate) * up is made on the way.  None for shapes it does not take."""
    if swiglu:
        a_parts, a_stride = _parts(a)
        M, K2 = a.shape[-2:]
        K = K2 // 2
        if a.dtype == torch.float32:
            mode = 1
        elif a.dtype == torch.bfloat16 and a_parts == 1:
            mode = 2
        else:
            return None
        lda = a.stride(-2)
    else:
        if a.dtype != torch.bfloat16 or a.dim() != 2:
            return None
        a_parts, a_stride, mode = 1, 0, 0
        M, K = a.shape
        lda = a.stride(0)
    N = w.shape[0]
    if not (w.dtype == torch.bfloat16 and 0 < M <= (SKINNY_MAX_ROWS if swiglu else LDS_MAX_ROWS) and K % 8 == 0
            and a.stride(-1) == 1 and lda % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and w.is_contiguous()
            and a_stride % 4 == 0):
        return None
    _dev(w, bias)
    _need(w.dim() == 2 and w.shape[1] == K, f"gemm: w must be [N, {K}], got {tuple(w.shape)}")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    lib = _lib()
    parts = lib.llogos_gemm_skinny_lds_parts(K, int(splits))
    if parts > 1:
        _need(bias is None, "gemm: a product in parts leaves the bias to its consumer")
        out_dtype = torch.float32
    out = torch.empty((parts, M, N), dtype=out_dtype, device=a.device)
    code = lib.llogos_gemm_skinny_lds_bf16(
        _p(out), _DT[out_dtype], _p(a), mode, lda, a_parts, ctypes.c_longlong(a_stride), _p(w), _p(bias),
        M, N, K, N, ctypes.c_longlong(M * N), int(splits), int(row_blocks), _stream())
    if code == -2:
        return None
    _check(code, "gemm_skinny_lds_bf16")
    return out


def gemm_strips_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                     splits: int, strips: int) -> Optional[torch.Tensor]:
    """The bfloat16 product for up to 128 rows whose operands go straight into LDS, several
    stages ahead, with blocks of `strips` 16-row strips of w: [parts, M, N], the same parts of k
    and the same sums as gemm_skinny_lds_bf16.  None for shapes it does not take."""
    if a.dtype != torch.bfloat16 or a.dim() != 2 or w.dtype != torch.bfloat16 or w.dim() != 2:
        return None
    M, K = a.shape
    N = w.shape[0]
    if not (0 < M <= LDS_MAX_ROWS and K % 64 == 0 and a.stride(1) == 1 and a.stride(0) % 8 == 0 and w.shape[1] == K
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and w.is_contiguous() and 2 <= strips <= 9):
        return None
    _dev(w, bias)
    _need(a.is_cuda and a.device == w.device, "gemm: a and w must be on the same GPU")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    lib = _lib()
    parts = lib.llogos_gemm_skinny_lds_parts(K, int(splits))
    if parts > 1:
        _need(bias is None, "gemm: a product in parts leaves the bias to its consumer")
        out_dtype = torch.float32
    out = torch.empty((parts, M, N), dtype=out_dtype, device=a.device)
    code = lib.llogos_gemm_strips_bf16(_p(out), _DT[out_dtype], _p(a), a.stride(0), _p(w), _p(bias), M, N, K, N,
                                       ctypes.c_longlong(M * N), int(splits), int(strips), _stream())
    if code == -2:
        return None
    _check(code, "gemm_strips_bf16")
    return out


class PackedWeight:
    """A bfloat16 matrix [N, K] in the order in which the matrix cores take it (pack_weights): blocks of
    64 rows, steps of 32 values of k, one 16-byte fragment a lane, zero-padded.  The few-row
    products stream it as one contiguous run per block."""
    __slots__ = ("data", "N", "K", "gate_rows")

    def __init__(self, data: torch.Tensor, N: int, K: int, gate_rows: int = 0):
        # gate_rows > 0: w is [gate; up] of gate_rows rows each and the packed strips of 16 rows alternate
        # between the two, for the product that makes silu(gate) * up in its epilogue (and for no other)
        self.data, self.N, self.K, self.gate_rows = data, N, K, gate_rows

    def rows(self, n: int) -> Optional["PackedWeight"]:
        """The first n rows as a packed matrix of their own (whole blocks of 64 rows only)."""
        if n == self.N:
            return self
        if n <= 0 or n > self.N or n % 64 or self.gate_rows:
            return None
        per_block = -(-self.K // 32) * 2048                  # bfloat16 elements of one block of rows
        return PackedWeight(self.data[: (n // 64) * per_block], n, self.K)


def packed_weight_bytes(N: int, K: int) -> int:
    return -(-N // 64) * -(-K // 32) * 4096


def pack_weights(w: torch.Tensor, gate_rows: int = 0) -> PackedWeight:
    """A packed copy of the bfloat16 matrix w [N, K].  gate_rows: w is a gate matrix on top of an up
    matrix of gate_rows rows each (a multiple of 16), and strips of 16 gate rows and of the 16 up
    rows of the same columns follow one another in the copy (see gemm_packed_gated_bf16)."""
    _dev(w)
    _need(w.dtype == torch.bfloat16 and w.dim() == 2, "pack_weights: w must be bfloat16 [N, K]")
    N, K = w.shape
    _need(gate_rows == 0 or (gate_rows % 16 == 0 and N == 2 * gate_rows), "pack_weights: gate and up of a multiple of 16 rows each")
    data = torch.empty(packed_weight_bytes(N, K) // 2, dtype=torch.bfloat16, device=w.device)
    _check(_lib().llogos_pack_weights(_p(data), _p(w), N, K, int(gate_rows), _stream()), "pack_weights")
    return PackedWeight(data, N, K, int(gate_rows))


def gemm_packed_gated_bf16(a: torch.Tensor, pw: PackedWeight, out_dtype: torch.dtype, chunk: int = 256) -> Optional[torch.Tensor]:
    """silu(a . gate^T) * (a . up^T) as [M, gate_rows] for up to 64 rows of bfloat16 activations, on a matrix
    packed with gate_rows: the gate/up product stays in registers.  None for shapes it does not take."""
    if pw.gate_rows <= 0 or a.dtype != torch.bfloat16 or a.dim() != 2:
        return None
    M, K = a.shape
    if not (K == pw.K and 0 < M <= SKINNY_MAX_ROWS and K % 8 == 0 and a.stride(1) == 1 and a.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and pw.data.data_ptr() % 16 == 0):
        return None
    _dev(pw.data)
    _need(a.is_cuda and a.device == pw.data.device, "gemm: a and w must be on the same GPU")
    out = torch.empty((M, pw.gate_rows), dtype=out_dtype, device=a.device)
    code = _lib().llogos_gemm_packed_gated_bf16(_p(out), _DT[out_dtype], _p(a), a.stride(0), _p(pw.data), M, pw.N, K,
                                                pw.gate_rows, int(chunk), _stream())
    if code == -2:
        return None
    _check(code, "gemm_packed_gated_bf16")
    return out


def packed_plan(M: int, N: int, K: int) -> Tuple[int, int]:
    """(blocks along k, values of k per LDS buffer) for the few-row product on packed weights: the
    blocks along k as for the row-major form (the same trade of evenness, enough blocks and the
    cost of partial sums, measured again on packed weights), and the shorter buffer for up to 16
    rows, where it was 2 to 5 % faster.  One plan per class of row count (16, 32, 64); the kernel itself
    works in tiles of 16 rows, 1 to 4 of them (33 to 48 rows take three: 41.7 us against 46.1 for the 8B
    gate/up matrix), which changes no sum."""
    return lds_splits(M, N, K), (128 if M <= 16 else 256)


def gemm_packed_bf16(a: torch.Tensor, pw: PackedWeight, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                     splits: int = 1, chunk: int = 256, swiglu: bool = False) -> Optional[torch.Tensor]:
    """The few-row bfloat16 product on packed weights: [parts, M, N]; parts > 1 are float32 partial
    sums over ranges of k that the consumer adds.  With `swiglu`, `a` is the fused gate/up product
    ([M, 2 K] bfloat16 or float32 partial sums [parts, M, 2 K]) and silu(gate) * up is made on the
    way.  None for shapes it does not take."""
    if swiglu:
        a_parts, a_stride = _parts(a)
        M, K2 = a.shape[-2:]
        K = K2 // 2
        if a.dtype == torch.float32:
            mode = 1
        elif a.dtype == torch.bfloat16 and a_parts == 1:
            mode = 2
        else:
            return None
        lda = a.stride(-2)
    else:
        if a.dtype != torch.bfloat16 or a.dim() != 2:
            return None
        a_parts, a_stride, mode = 1, 0, 0
        M, K = a.shape
        lda = a.stride(0)
    N = pw.N
    if not (K == pw.K and 0 < M <= SKINNY_MAX_ROWS and K % 8 == 0 and a.stride(-1) == 1 and lda % 8 == 0
            and a.data_ptr() % 16 == 0 and pw.data.data_ptr() % 16 == 0 and a_stride % 4 == 0):
        return None
    _dev(pw.data, bias)
    _need(a.is_cuda and a.device == pw.data.device, "gemm: a and w must be on the same GPU")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    lib = _lib()
    parts = lib.llogos_gemm_packed_parts(K, int(splits), int(chunk))
    _need(parts >= 1, "gemm: the LDS buffer holds 128 or 256 values of k")
    if parts > 1:
        _need(bias is None, "gemm: a product in parts leaves the bias to its consumer")
        out_dtype = torch.float32
    out = torch.empty((parts, M, N), dtype=out_dtype, device=a.device)
    code = lib.llogos_gemm_packed_bf16(
        _p(out), _DT[out_dtype], _p(a), mode, lda, a_parts, ctypes.c_longlong(a_stride), _p(pw.data), _p(bias),
        M, N, K, N, ctypes.c_longlong(M * N), int(splits), int(chunk), _stream())
    if code == -2:
        return None
    _check(code, "gemm_packed_bf16")
    return out


RESIDUAL_MAX_ROWS = 16     # rows at most of the product that adds itself to the residual stream
# "on" (the default): steps of up to 16 rows close a mixer and a feed-forward with gemm_residual_bf16 and
# open the next with gemm_packed_unscaled_bf16 where the shapes allow; "off": the products in parts and
# the norm's own kernel everywhere.  LLOGOS_RESIDUAL_PRODUCT in the environment sets the default.
RESIDUAL_PRODUCT = os.environ.get("LLOGOS_RESIDUAL_PRODUCT", "on")


@dataclass
class RowSquares:
    """What a product that has added itself to the residual stream x leaves beside it: sums [blocks, 16],
    float32, each of the product's blocks holding for each row of x the sum of the squares of its 16 or 32
    columns.  A norm over the rows of x needs no other pass over them (gemm_packed_unscaled_bf16)."""
    sums: Optional[torch.Tensor]                # None: the product left nothing but the complete stream
    width: int                                  # columns of x that the sums cover
    unscaled: Optional[torch.Tensor] = None     # bfloat16 [M, width]: x * norm_w, the rmsnorm's rows without their scale
    norm_w: Optional[torch.Tensor] = None       # the weight that `unscaled` was made with


def residual_plan(M: int, N: int, K: int, n_cus: Optional[int] = None) -> Tuple[int, int]:
    """(waves of a block, strips of 16 rows of w a block) of gemm_residual_bf16; (0, 0): not served (then the
    product in parts over k and the norm's own kernel do the work).  A block owns its rows of w and all of k,
    and a compute unit streams what its blocks own at a bounded rate: the blocks have to fill the units evenly,
    one block a unit at best.  Measured on the MI355X (256 units) at 1, 8 and 16 rows against the product in
    parts plus the norm kernel (us):
      N / 16 <= units (1B, 3B, 8B widths): blocks of one strip, 8 waves: 8B o 9.0 against 12.4, down 21.0
        against 24.2 (two strips a block: 10.5 and 27.8: half the units idle);
      more strips than units: two strips a block, which share a wave's copy of the activations: 70B (256
        blocks) o 24.2 against 27.5, down 71.2 against 79.4 (one strip a block, two blocks a unit: 76.1); 14B
        (160 blocks) o 12.8 against 16.1; its down projection, 89 M weights on 160 of 256 units, only up to 4
        rows (31.6 against 35.4 at one row, 34.6 against 33.6 at 8, 38.4 against 34.1 at 16)."""
    if RESIDUAL_PRODUCT != "on" or not (0 < M <= RESIDUAL_MAX_ROWS and K % 8 == 0):
        return 0, 0
    n_cus = n_cus or compute_units()
    strips = -(-N // 16)
    waves = 8 if K >= 1024 else 4
    if N * K <= (1 << 22):                    # so small that only the number of kernels counts
        return waves, 1
    if strips <= n_cus:
        return (waves, 1) if strips >= n_cus // 2 else (0, 0)
    blocks = -(-strips // 2)
    if blocks < (3 * n_cus) // 4 and N * K > (1 << 25) and M > 4:
        return 0, 0
    return 8, 2


def gemm_residual_bf16(x: torch.Tensor, a: torch.Tensor, pw: PackedWeight, bias: Optional[torch.Tensor],
                       waves: int, norm_w: Optional[torch.Tensor] = None, strips: int = 1) -> Optional[RowSquares]:
    """x [M, N] (float32, in place) += a [M, K] . w^T (+ bias) for up to 16 rows of bfloat16 activations in
    one kernel, every sum in an order fixed by the shapes; returns the sums of squares of x's new rows, by
    strips of 16 columns, and with `norm_w` [N] also x * norm_w in bfloat16 (the rows of the rmsnorm with
    that weight, without their scale).  None for shapes it does not take."""
    if a.dtype != torch.bfloat16 or a.dim() != 2 or x.dim() != 2 or x.dtype != torch.float32 or pw.gate_rows:
        return None
    M, K = a.shape
    N = pw.N
    if not (K == pw.K and x.shape == (M, N) and 0 < M <= RESIDUAL_MAX_ROWS and K % 8 == 0 and a.stride(1) == 1
            and a.stride(0) % 8 == 0 and x.stride(1) == 1 and a.data_ptr() % 16 == 0 and pw.data.data_ptr() % 16 == 0):
        return None
    _dev(x, a, pw.data, bias, norm_w)
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    unscaled = None
    if norm_w is not None:
        _need(norm_w.dtype == torch.float32 and norm_w.shape == (N,) and norm_w.is_contiguous(), "gemm: norm weight must be float32 [N]")
        unscaled = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    sums = torch.empty((-(-(-(-N // 16)) // int(strips)), 16), dtype=torch.float32, device=x.device)
    code = _lib().llogos_gemm_residual_bf16(_p(x), x.stride(0), _p(sums), _p(unscaled), N, _p(norm_w), _p(a), a.stride(0),
                                            _p(pw.data), _p(bias), M, N, K, int(waves), int(strips), _stream())
    if code == -2:
        return None
    _check(code, "gemm_residual_bf16")
    return RowSquares(sums, N, unscaled, norm_w)


def gemm_packed_unscaled_bf16(squares: RowSquares, eps: float, pw: PackedWeight, bias: Optional[torch.Tensor],
                              out_dtype: torch.dtype, splits: int = 1, chunk: int = 128) -> Optional[torch.Tensor]:
    """The few-row product on packed weights with an rmsnorm's rows as its activations, of which `squares`
    holds x * norm_w in bfloat16 and the sums of squares of x (gemm_residual_bf16 with norm_w): the rows'
    scale 1 / sqrt(mean square + eps) is applied to the product, in float32.  On a matrix packed with
    gate_rows the result is silu(gate) * up [M, gate_rows], otherwise [parts, M, N] as gemm_packed_bf16 (a
    bias is added after the scale).  None for shapes it does not take."""
    a = squares.unscaled
    if a is None:
        return None
    M, K = a.shape
    N = pw.N
    if not (K == pw.K and squares.width == K and 0 < M <= RESIDUAL_MAX_ROWS and K % 8 == 0 and a.stride(1) == 1
            and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and pw.data.data_ptr() % 16 == 0):
        return None
    _dev(a, squares.sums, pw.data, bias)
    _need(squares.sums.dtype == torch.float32 and squares.sums.dim() == 2 and squares.sums.shape[1] == RESIDUAL_MAX_ROWS
          and squares.sums.is_contiguous() and squares.sums.shape[0] >= 1 and a.dtype == torch.bfloat16,
          "gemm: the sums of squares are float32 [parts, 16], the unscaled rows bfloat16")
    lib = _lib()
    gated = pw.gate_rows > 0
    if gated:
        if bias is not None:
            return None
        parts, cols = 1, pw.gate_rows
        out = torch.empty((M, cols), dtype=out_dtype, device=a.device)
    else:
        if bias is not None:
            _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
        parts = lib.llogos_gemm_packed_parts(K, int(splits), int(chunk))
        _need(parts >= 1, "gemm: the LDS buffer holds 128 or 256 values of k")
        if parts > 1:
            _need(bias is None, "gemm: a product in parts leaves the bias to its consumer")
            out_dtype = torch.float32
        cols = N
        out = torch.empty((parts, M, N), dtype=out_dtype, device=a.device)
    code = lib.llogos_gemm_packed_unscaled_bf16(
        _p(out), _DT[out_dtype], _p(a), a.stride(0), _p(squares.sums), squares.sums.shape[0], K,
        ctypes.c_float(eps), _p(pw.data), _p(bias), M, N, K, cols, ctypes.c_longlong(M * N), int(splits), int(chunk),
        int(gated), _stream())
    if code == -2:
        return None
    _check(code, "gemm_packed_unscaled_bf16")
    return out


# Which product serves many rows of bfloat16 (prompts): "auto" (the default): the hand-written tiled
# product (gemm_tiles_bf16 on the packed copy) where it was measured faster than the library's, which is
# the gate/up product with its SwiGLU epilogue from TILES_MIN_ROWS rows on, and the library's product
# elsewhere (as the reference uses a library there); "tiles": the hand-written one wherever it applies;
# "library": the library's everywhere.  LLOGOS_PROMPT_PRODUCT in the environment sets the default.
PROMPT_PRODUCT = os.environ.get("LLOGOS_PROMPT_PRODUCT", "auto")
TILES_MIN_ROWS, TILES_MAX_ROWS, TILES_MAX_K = 1024, 2048, 5120


def tiles_serve_gated(M: int, K: int = 0) -> bool:
    """Whether the tiled product makes silu(gate) * up for M rows of K values (rather than the library's product
    and a SwiGLU pass): by default from TILES_MIN_ROWS to TILES_MAX_ROWS rows with k up to TILES_MAX_K, where
    it was measured level or ahead (tiled against library + SwiGLU, us, sustained: 1B 63 / 67 at 1,024 rows,
    119 / 120 at 2,048; 8B 225 / 217 and 405 / 391, level inside the model; 14B 343 / 413 and 614 / 630).
    The library gains with the rows and with k (8B: 1.11 PFLOP/s at 1,024 rows, 1.34 from 4,096 on; 70B 1.41
    to 1.47) where the tiled product stays at 1.2: 8B at 4,096 rows 825 / 727, 70B at 2,048 rows 1,516 / 1,363,
    a 16,384-token prompt of the 8B sizes 278 ms against 268."""
    if PROMPT_PRODUCT == "tiles":
        return True
    return PROMPT_PRODUCT == "auto" and TILES_MIN_ROWS <= M <= TILES_MAX_ROWS and K <= TILES_MAX_K


def tiles_plan(M: int, N: int, K: int) -> Optional[Tuple[int, int]]:
    """(parts of k, token_tiles) with which the tiled product serves a plain product of M rows, or None where
    the library's does.  Measured on the MI355X at the layer sizes of 8B, 14B and 70B models: a matrix that
    is much longer than high (a feed-forward's down projection) with 129 to 1,024 rows of activations is where
    the library is furthest from its best (14B, 256 rows: 119 us against 65; 70B: 291 against 143; 8B, 512 rows:
    88 against 68), and blocks along k fill the compute units that its few row tiles leave idle.  Elsewhere
    the library's product was level or ahead (by 10 to 25 % from 2,048 rows on)."""
    if PROMPT_PRODUCT == "library" or M <= SKINNY_MAX_ROWS or K % 64:
        return None
    if PROMPT_PRODUCT == "tiles":
        return 1, 0
    if K >= 2 * N and LDS_MAX_ROWS < M <= 1024:
        parts, token_tiles = (4, 2) if M <= 256 else ((4, 0) if M <= 512 else (2, 0))
        while parts > 1 and (K // 64) // parts < 2:
            parts //= 2
        return parts, token_tiles
    return None


def gemm_tiles_bf16(a: torch.Tensor, pw: PackedWeight, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                    parts: int = 1, token_tiles: int = 0) -> Optional[torch.Tensor]:
    """a [M, K] . w^T on the packed copy of w for any number of rows (tiles of 256 or 128 tokens x 256 rows,
    v_mfma_f32_32x32x16_bf16): [M, N] with the bias added, or, for a matrix packed with gate_rows,
    [M, gate_rows] = silu(gate) * up; with parts > 1 float32 partial sums [parts, M, N] over ranges of k.
    token_tiles: 4 or 2 force tiles of 256 or 128 tokens, 0 lets the launch choose.
    None for shapes it does not take (K no multiple of 64, parts of fewer than 128 values of k)."""
    if a.dtype != torch.bfloat16 or a.dim() != 2:
        return None
    M, K = a.shape
    if not (K == pw.K and M > 0 and K % 64 == 0 and a.stride(1) == 1 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0):
        return None
    gated = pw.gate_rows > 0
    _dev(pw.data, bias)
    _need(a.is_cuda and a.device == pw.data.device, "gemm: a and w must be on the same GPU")
    _need(not (gated and bias is not None), "gemm: the gated product takes no bias")
    _need(parts >= 1 and not (gated and parts > 1), "gemm: the gated product comes in one part")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (pw.N,), "gemm: bias must be float32 [N]")
        _need(parts == 1, "gemm: a product in parts leaves the bias to its consumer")
    if parts > 1:
        out_dtype = torch.float32
    width = pw.gate_rows if gated else pw.N
    out = torch.empty((parts, M, width), dtype=out_dtype, device=a.device)
    code = _lib().llogos_gemm_tiles_bf16(_p(out), _DT[out_dtype], _p(a), a.stride(0), _p(pw.data), _p(bias), M, pw.N, K,
                                         width, ctypes.c_longlong(M * width), int(gated), int(parts), int(token_tiles),
                                         compute_units(a.device), _stream())
    if code == -2:
        return None
    _check(code, "gemm_tiles_bf16")
    return out[0] if parts == 1 else out


def gemm_product(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, swiglu_input: bool = False,
                 f32_ok: bool = False, packed: Optional[PackedWeight] = None) -> torch.Tensor:
    """a [M, K] . w [N, K]^T without bias, as [M, N] of `out_dtype` or as float32 partial sums
    [parts, M, N] for a consumer that adds them (rmsnorm, qk_rope_cache, swiglu, sum_parts).
    With `swiglu_input`, `a` is a fused gate/up product ([M, 2 K] or parts of it) and the
    product is taken of silu(gate) * up.  With `f32_ok` the consumer also takes one float32
    [M, N], which spares the result a rounding to bfloat16.

    float32 operands: plain FMAs in 32-bit throughout.  bfloat16 operands: up to 64 rows the
    hand-written weight-streaming kernels (on the packed copy of w when there is one: `packed`),
    up to 128 rows too where w is much longer than it has rows (see long_inner); for more rows the
    hand-written tiled product where it was measured ahead (see tiles_plan); otherwise the
    library product (as the reference uses a library for its prompt products,
    Daisi.Llogos.Cuda/CudaBackend.cs:158-316)."""
    M = a.shape[-2]
    if packed is not None and packed.gate_rows:
        packed = None                                       # its rows are in another order: only the gated product reads it
    if packed is not None and w.dtype == torch.bfloat16 and M <= SKINNY_MAX_ROWS and out_dtype == torch.bfloat16:
        splits, chunk = packed_plan(M, packed.N, packed.K)
        src, fused = a, swiglu_input
        # silu(gate) * up inside the product costs every block of rows of w a second read of the
        # gate/up row: worth it for few rows in bfloat16, not for partial sums or many rows
        if fused and not (M <= 16 and a.dtype == torch.bfloat16 and (a.dim() == 2 or a.shape[0] == 1)):
            src, fused = swiglu(a, out_dtype), False
        if not fused and src.dim() == 3 and src.shape[0] == 1:
            src = src[0]
        out = gemm_packed_bf16(src, packed, None, torch.float32 if f32_ok else out_dtype, splits, chunk, fused)
        if out is not None:
            return out
    if w.dtype == torch.bfloat16 and M <= SKINNY_MAX_ROWS and out_dtype == torch.bfloat16:
        few_dtype = torch.float32 if f32_ok else out_dtype              # what a product in one part is written as
        kernel, splits, row_blocks = skinny_plan(M, w.shape[0], w.shape[1])
        if kernel == "stationary" and not swiglu_input and a.dim() == 2:
            out = gemm_skinny_stationary_bf16(a, w, None, few_dtype, row_blocks)
            if out is not None:
                return out
            kernel, splits, row_blocks = "lds", 1, 1
        elif kernel == "stationary":
            kernel, splits, row_blocks = "lds", 1, 1
        if kernel == "strips":
            if swiglu_input:
                a, swiglu_input = swiglu(a, out_dtype), False
            out = gemm_strips_bf16(a, w, None, few_dtype, splits, row_blocks) if a.dim() == 2 else None
            if out is not None:
                return out
            kernel, splits, row_blocks = "lds", lds_splits(M, w.shape[0], w.shape[1]), 1
        # silu(gate) * up inside the product costs every block of rows of w a second read of the
        # gate/up row: worth it for few rows in bfloat16, not for partial sums or many rows
        if swiglu_input and not (M <= 16 and a.dtype == torch.bfloat16 and (a.dim() == 2 or a.shape[0] == 1)):
            a, swiglu_input = swiglu(a, out_dtype), False
        if swiglu_input or kernel == "lds":
            out = gemm_skinny_lds_bf16(a, w, None, few_dtype, splits if kernel == "lds" else 1, row_blocks,
                                       swiglu_input)
            if out is not None:
                return out
        if not swiglu_input and a.dtype == torch.bfloat16:
            out = gemm_skinny_bf16(a, w, None, few_dtype, splits if kernel == "regs" else 1, row_blocks)
            if out is not None:
                return out
    if swiglu_input:
        a = swiglu(a, out_dtype)
    if SKINNY_MAX_ROWS < M <= LDS_MAX_ROWS and long_inner(w) and a.dtype == torch.bfloat16 and out_dtype == torch.bfloat16:
        out = gemm_skinny_lds_bf16(a, w, None, torch.float32 if f32_ok else out_dtype,
                                   lds_splits(M, w.shape[0], w.shape[1]), 1)
        if out is not None:
            return out
    plan = tiles_plan(M, packed.N, packed.K) if packed is not None else None
    if plan is not None and out_dtype == torch.bfloat16 and a.dtype == torch.bfloat16 and a.dim() == 2:
        out = gemm_tiles_bf16(a, packed, None, torch.float32 if f32_ok else out_dtype, parts=plan[0], token_tiles=plan[1])
        if out is not None:
            return out
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out_dtype == torch.bfloat16 and a.is_contiguous() \
            and M > SKINNY_MAX_ROWS:
        if f32_ok:
            return torch.mm(a, w.t(), out_dtype=torch.float32)
        return torch.matmul(a, w.t())
    return gemm_generic(a, w, None, out_dtype)


def gemm_library_add(x: torch.Tensor, a: torch.Tensor, w: torch.Tensor, packed: Optional[PackedWeight] = None) -> bool:
    """x [M, N] (float32, in place) += a [M, K] . w^T by the library's bfloat16 product with float32
    accumulation and the sum in its epilogue, where the library serves this product anyway (prompts of
    more than 128 rows that the tiled product does not take): the stream is read and written once there
    instead of the product being written, read again and added by the norm's kernel.  False (and x
    untouched) otherwise.  The result is the float32 product added to x, bit for bit."""
    if RESIDUAL_PRODUCT != "on":
        return False
    if not (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dtype == torch.float32 and a.dim() == 2
            and x.dim() == 2 and a.is_contiguous() and x.is_contiguous() and w.is_contiguous()):
        return False
    M, N = a.shape[0], w.shape[0]
    if M <= LDS_MAX_ROWS or x.shape != (M, N) or a.shape[1] != w.shape[1] or a.shape[1] % 8:
        return False
    if packed is not None and tiles_plan(M, packed.N, packed.K) is not None:
        return False
    torch.addmm(x, a, w.t(), out_dtype=torch.float32, out=x)
    return True


def gemm(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
         packed: Optional[PackedWeight] = None) -> torch.Tensor:
    """a [M, K] . w [N, K]^T (+ bias [N]) -> one plain [M, N] tensor of `out_dtype`."""
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        M = a.shape[0]
        if packed is not None and not packed.gate_rows and M <= SKINNY_MAX_ROWS:
            out = gemm_packed_bf16(a, packed, bias, out_dtype, 1, packed_plan(M, packed.N, packed.K)[1])
            if out is not None:
                return out[0]
        if M <= SKINNY_MAX_ROWS:
            kernel, _, row_blocks = skinny_plan(M, w.shape[0], w.shape[1])
            if kernel == "stationary":
                out = gemm_skinny_stationary_bf16(a, w, bias, out_dtype, row_blocks)
                kernel, row_blocks = "lds", 1
            elif kernel == "strips":
                out = gemm_strips_bf16(a, w, bias, out_dtype, 1, row_blocks)
                kernel, row_blocks = "lds", 1
            else:
                out = None
            if out is None:
                fn = gemm_skinny_lds_bf16 if kernel == "lds" else gemm_skinny_bf16
                out = fn(a, w, bias, out_dtype, 1, row_blocks)
            if out is not None:
                return out[0]
        elif out_dtype == torch.bfloat16 and a.is_contiguous():
            out = torch.matmul(a, w.t())
            if bias is not None:
                out += bias.to(torch.bfloat16)
            return out
        elif out_dtype == torch.float32 and a.is_contiguous() and a.shape[1] % 8 == 0:
            # float32 results for many rows (the logits of many positions): the library's product
            # with float32 accumulation and output, one pass over w
            out = torch.mm(a, w.t(), out_dtype=torch.float32)
            if bias is not None:
                out += bias
            return out
    return gemm_generic(a, w, bias, out_dtype)


_attn_workspaces = {}
PREFILL_TILE_ROWS = 0        # 0: chosen by the step; 64 or 128 force a prefill attention kernel (tests)
PREFILL_HALVES = 0           # 0: chosen by the step; 1 or 2 sets of waves a block of the 128-row kernel (tests)


def prefill_halves(lens: Sequence[int], starts: Optional[Sequence[int]], n_heads: int, n_cus: Optional[int] = None) -> int:
    """Sets of waves a block of the 128-row prompt attention: 2 (the sets take a tile's pages in
    turn) where the pages of the longest tile, one after the other, take longer than the chip
    needs for all tiles; 1 (two independent blocks a compute unit, 15 % more throughput) where
    the work of all tiles decides.  Measured at the 8B head shape: two sets win up to 2,048
    tokens of one prompt (1,536: 45 us against 57) and lose from 2,560 on and for many short
    prompts."""
    n_cus = n_cus or compute_units()
    longest = total = 0
    for i, n in enumerate(lens):
        start = starts[i] if starts else 0
        for t in range(0, n, 128):
            pages = (start + min(n, t + 128) + PAGE_TOKENS - 1) // PAGE_TOKENS
            longest = max(longest, pages)
            total += pages
    return 2 if longest * 2 * n_cus > 1.7 * total * n_heads else 1


def _attn_workspace(device: torch.device, floats: int) -> torch.Tensor:
    """Scratch memory of the decode attention, at least `floats` long.  A workspace that has
    become too small stays alive beside its successor: captured steps keep its address."""
    key = (device.type, device.index)
    held = _attn_workspaces.setdefault(key, [])
    if not held or held[-1].numel() < floats:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("attention workspace must be made before a step is captured")
        size = max(floats, 1 << 20, 2 * held[-1].numel() if held else 0)
        held.append(torch.empty(size, dtype=torch.float32, device=device))
    return held[-1]


def attention_mfma_bf16(ctx, q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                        table: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                        window: int = 0, sinks: int = 0) -> Optional[torch.Tensor]:
    """bfloat16 attention on the matrix cores; None for shapes it does not take (head sizes
    other than 64 and 128, more than 16 query heads per kv head)."""
    if q.dtype != torch.bfloat16 or head_dim not in (64, 128) or n_heads // n_kv_heads > 16:
        return None
    if q_stride % 8 or q.data_ptr() % 16:
        return None
    _dev(k_pool, v_pool, table)
    _i32(table, "table")
    _check_pools(k_pool, v_pool, n_kv_heads, head_dim, "attention")
    _need(k_pool.dtype == torch.bfloat16, "attention: q and cache types differ")
    T = ctx.n_tokens
    _need(q.numel() >= (T - 1) * q_stride + n_heads * head_dim, "attention: q too small")
    out = torch.empty((T, n_heads * head_dim), dtype=torch.bfloat16, device=q.device)
    lib = _lib()
    if ctx.is_decode:
        width = table.shape[1]
        floats = lib.llogos_attn_decode_workspace(T, n_heads, n_kv_heads, head_dim, width)
        ws = _attn_workspace(q.device, floats)
        code = lib.llogos_attn_decode_bf16(
            _p(out), _p(q), q_stride, _p(k_pool), _p(v_pool), _p(table), table.stride(0), width, _p(ctx.tok_pos),
            T, n_heads, n_kv_heads, head_dim, ctypes.c_float(scale), window, sinks, _p(ws),
            ctypes.c_longlong(ws.numel()), _stream())
    else:
        cu = ctx.cu_dev
        _need(cu is not None and cu.numel() == ctx.batch + 1, "attention: the step's token offsets are missing")
        # long sequences: tiles of 128 tokens whose waves share each page through LDS; short
        # ones: tiles of 64 whose waves read the pages themselves
        lens = [ctx.cu_seqlens[i + 1] - ctx.cu_seqlens[i] for i in range(ctx.batch)]
        tile_rows = PREFILL_TILE_ROWS or (128 if max(lens) > 64 else 64)
        n_tiles = sum(-(-n // tile_rows) for n in lens)
        halves = PREFILL_HALVES or (prefill_halves(lens, getattr(ctx, "starts", None), n_heads) if tile_rows == 128 else 1)
        code = lib.llogos_attn_prefill_bf16(
            _p(out), _p(q), q_stride, _p(k_pool), _p(v_pool), _p(table), table.stride(0), _p(cu), _p(ctx.tok_pos),
            ctx.batch, n_tiles, tile_rows, n_heads, n_kv_heads, head_dim, ctypes.c_float(scale), window, sinks,
            halves, _stream())
    if code == -2:
        return None
    _check(code, "attention_mfma_bf16")
    return out


def attention_decode_fused(ctx, qkv: torch.Tensor, bias: Optional[torch.Tensor], n_heads: int, n_kv_heads: int,
                           head_dim: int, rot: int, pairing: int, q_norm_w: Optional[torch.Tensor],
                           k_norm_w: Optional[torch.Tensor], eps: float, cs: torch.Tensor, k_pool: torch.Tensor,
                           v_pool: torch.Tensor, table: torch.Tensor, scale: float, window: int = 0,
                           sinks: int = 0) -> Optional[torch.Tensor]:
    """A single-token step's attention straight from the fused projection rows [q | k | v]
    (float32 [T, W] or partial sums [parts, T, W]): bias, per-head norm, rotation and the cache
    write happen inside the attention kernel.  For bfloat16 caches, head sizes 64 and 128 rotated
    whole with split-half pairing; None for anything else (the caller then runs the steps apart)."""
    if not (ctx.is_decode and qkv.dtype == torch.float32 and k_pool.dtype == torch.bfloat16 and head_dim in (64, 128)
            and rot == head_dim and pairing == 0 and n_heads % n_kv_heads == 0 and n_heads // n_kv_heads <= 16):
        return None
    parts, part_stride = _parts(qkv)
    T = qkv.shape[-2]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    if qkv.stride(-1) != 1 or qkv.stride(-2) % 2 or part_stride % 2 or qkv.data_ptr() % 8:
        return None
    _dev(qkv, bias, q_norm_w, k_norm_w, cs, k_pool, v_pool, table, ctx.tok_pos)
    _i32(table, "table"); _i32(ctx.tok_pos, "tok_pos")
    _need(T == ctx.n_tokens == ctx.batch and qkv.shape[-1] == width, f"attention: qkv must be [{ctx.batch}, {width}]")
    _need(cs.dtype == torch.float32 and cs.shape == (T, rot // 2, 2) and cs.is_contiguous(), "attention: rotary table shape")
    _need(table.dim() == 2 and table.shape[0] == T and ctx.tok_pos.numel() == T, "attention: one table row and position a sequence")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (width,), f"attention: bias must be float32 [{width}]")
    for wgt in (q_norm_w, k_norm_w):
        if wgt is not None:
            _need(wgt.dtype == torch.float32 and wgt.shape == (head_dim,), "attention: norm weight float32 [head_dim]")
    _check_pools(k_pool, v_pool, n_kv_heads, head_dim, "attention")
    _need(v_pool.dtype == torch.bfloat16, "attention: cache types differ")
    out = torch.empty((T, n_heads * head_dim), dtype=torch.bfloat16, device=qkv.device)
    lib = _lib()
    width_pages = table.shape[1]
    ws = _attn_workspace(qkv.device, lib.llogos_attn_decode_workspace(T, n_heads, n_kv_heads, head_dim, width_pages))
    code = lib.llogos_attn_decode_fused_bf16(
        _p(out), _p(qkv), parts, ctypes.c_longlong(part_stride), qkv.stride(-2), _p(bias), _p(q_norm_w), _p(k_norm_w),
        ctypes.c_float(eps), _p(cs), _p(k_pool), _p(v_pool), _p(table), table.stride(0), width_pages, _p(ctx.tok_pos),
        T, n_heads, n_kv_heads, head_dim, ctypes.c_float(scale), window, sinks, _p(ws),
        ctypes.c_longlong(ws.numel()), _stream())
    if code == -2:
        return None
    _check(code, "attention_decode_fused")
    return out


def attention(ctx, q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
              table: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
              window: int = 0, sinks: int = 0) -> torch.Tensor:
    """Attention of the step's query rows over the cache pages of their sequences."""
    if q.dtype == torch.bfloat16:
        out = attention_mfma_bf16(ctx, q, q_stride, k_pool, v_pool, table, n_heads, n_kv_heads, head_dim, scale,
                                  window, sinks)
        if out is not None:
            return out
    return attention_generic(q, q_stride, k_pool, v_pool, table, ctx.tok_seq, ctx.tok_pos,
                             n_heads, n_kv_heads, head_dim, scale, window, sinks)


# ----------------------------------------------------------------------------
# sampling
# ----------------------------------------------------------------------------
def sample_prepare(logits: torch.Tensor, history: Optional[torch.Tensor], history_len: Optional[torch.Tensor],
                   repetition: float, frequency: float, presence: float, temperature: float,
                   penalize_newline: bool, banned: Sequence[int] = ()) -> torch.Tensor:
    """A copy of float32 logits [R, V] with penalties over each row's recent tokens
    (`history` int32 [R, W], `history_len` int32 [R]), banned ids at -inf, times 1/temperature."""
    _dev(logits, history, history_len)
    _i32(history, "history"); _i32(history_len, "history_len")
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "sample_prepare: logits must be float32 [R, V]")
    _need(len(banned) <= MAX_BANNED, f"sample_prepare: at most {MAX_BANNED} banned ids, got {len(banned)}")
    R, V = logits.shape
    if history is not None:
        _need(history.dim() == 2 and history.shape[0] == R and history_len is not None
              and history_len.numel() == R, "sample_prepare: history [R, W] with lengths [R]")
    work = torch.empty_like(logits)
    ban = (ctypes.c_int * MAX_BANNED)(*list(banned))
    inv_t = 1.0 / temperature if temperature > 0 else 1.0
    _check(_lib().llogos_sample_prepare(
        _p(work), _p(logits), R, V, _p(history), _p(history_len), history.stride(0) if history is not None else 0,
        ctypes.c_float(repetition), ctypes.c_float(frequency), ctypes.c_float(presence), ctypes.c_float(inv_t),
        int(penalize_newline), ban, len(banned), _stream()), "sample_prepare")
    return work


SAMPLE_ORDERS = {"single": 0, "head": 1, "whole": 2}


def sample_pipeline(work: torch.Tensor, uniforms: torch.Tensor, top_k: int, top_p: float, min_p: float,
                    typical_p: float, min_keep: int, order: str = "head") -> torch.Tensor:
    """Token ids int32 [R] drawn from prepared rows `work` with one uniform number per row:
    top-k, min-p, softmax, typical-p, top-p, draw.  order "head": a row is first tried with
    the head of its descending order alone (a histogram finds it; no sort of the vocabulary),
    and rows that this cannot decide are sorted whole by many blocks; "whole": every row is
    sorted so; "single": every row is sorted by its own block (slow, the plain form).  Rows
    sorted whole are overwritten with probabilities."""
    _dev(work, uniforms)
    _need(work.dtype == torch.float32 and work.dim() == 2, "sample_pipeline: work must be float32 [R, V]")
    _need(order in SAMPLE_ORDERS, f"sample_pipeline: order must be one of {sorted(SAMPLE_ORDERS)}")
    R, V = work.shape
    _need(uniforms.dtype == torch.float32 and uniforms.numel() == R, "sample_pipeline: one float32 uniform per row")
    n_pad = 1
    while n_pad < V:
        n_pad <<= 1
    scratch = torch.empty((R, n_pad), dtype=torch.int64, device=work.device)
    prob = torch.empty_like(work) if order == "head" else None
    out = torch.empty((R,), dtype=torch.int32, device=work.device)
    _check(_lib().llogos_sample_pipeline(
        _p(out), _p(work), _p(prob), R, V, _p(scratch), n_pad, _p(uniforms), int(top_k), ctypes.c_float(top_p),
        ctypes.c_float(min_p), ctypes.c_float(typical_p), int(min_keep), SAMPLE_ORDERS[order], _stream()),
        "sample_pipeline")
    return out


# ----------------------------------------------------------------------------
# what the GPU does at best, measured
# ----------------------------------------------------------------------------
def measure_read_bandwidth(n_bytes: int, repeats: int = 20, blocks_per_unit: int = 8, device="cuda:0") -> float:
    """Bytes a second at which a kernel that only reads streams `n_bytes` of device memory
    (16-byte loads that do not stay in the caches, 32 KB of consecutive memory a block and round),
    best of `repeats` runs over a buffer that was not the last thing read."""
    dev = torch.device(device)
    n_bytes = max(1 << 20, n_bytes // 16 * 16)
    with torch.cuda.device(dev):
        buf = torch.empty(n_bytes // 4, dtype=torch.int32, device=dev).fill_(1)
        other = torch.empty(max(n_bytes // 4, 1 << 27), dtype=torch.int32, device=dev).fill_(2)   # evicts the caches
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        blocks = compute_units(dev) * blocks_per_unit
        lib, best = _lib(), 0.0
        for _ in range(repeats):
            _check(lib.llogos_measure_read(_p(other), ctypes.c_longlong(other.numel() * 4), blocks, _p(sink), _stream()), "measure_read")
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            _check(lib.llogos_measure_read(_p(buf), ctypes.c_longlong(n_bytes), blocks, _p(sink), _stream()), "measure_read")
            end.record()
            end.synchronize()
            best = max(best, n_bytes / (start.elapsed_time(end) * 1e-3))
    return best


def measure_mfma_rate(iters: int = 20000, blocks_per_unit: int = 2, device="cuda:0", noisy: bool = True,
                      shapes=(16, 32)) -> float:
    """bfloat16 flops a second of MFMAs issued back to back by eight waves on every compute unit
    (independent accumulators): the better of v_mfma_f32_16x16x32_bf16 and v_mfma_f32_32x32x16_bf16.
    noisy: operands of random values, as real data is (the chip clocks lower under their power than
    with the few small constants of noisy=False)."""
    dev = torch.device(device)
    with torch.cuda.device(dev):
        blocks = compute_units(dev) * blocks_per_unit
        out = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
        lib, best = _lib(), 0.0
        for shape in tuple(shapes) * 2:
            per_iter = 8 * 16384.0 if shape == 16 else 4 * 32768.0
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            _check(lib.llogos_measure_mfma(_p(out), blocks, iters, shape, int(noisy), _stream()), "measure_mfma")
            end.record()
            end.synchronize()
            best = max(best, blocks * 4 * iters * per_iter / (start.elapsed_time(end) * 1e-3))
    return best
