"""Matrix products with checkpoint matrices: y = x . W^T (+ b), W stored [out, in]
(reference: Daisi.Llogos/Inference/ForwardPass.cs:890-895)."""
from __future__ import annotations

from typing import Callable, List, Optional, Sequence

import torch

from ..ops import kernels as K
from .base import NormedRows, Part, Residual, Runtime, TensorSpec


class Linear(Part):
    """One or several checkpoint matrices applied as one product.  Several matrices with
    the same input width are stacked by rows at bind time ([Wq; Wk; Wv], [Wgate; Wup]), so
    the output row is the concatenation of their outputs."""

    def __init__(self, names: Sequence[str], in_features: int, out_features: Sequence[int],
                 bias: bool = False, suffix: str = ".weight", gated: bool = False):
        # gated: the two stacked matrices are a gate and an up projection whose product is only ever
        # wanted as silu(gate) * up; their packed copy then serves the product that makes that in its
        # epilogue (gated_product)
        self.gated = bool(gated) and len(out_features) == 2 and out_features[0] == out_features[1] \
            and out_features[0] % 16 == 0 and not bias
        self.names = list(names)
        self.in_features = in_features
        self.out_features = list(out_features)
        self.has_bias = bias
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.packed: Optional[K.PackedWeight] = None     # the copy that steps of up to 64 rows stream

    @property
    def total_out(self) -> int:
        return sum(self.out_features)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = []
        for n, o in zip(self.names, self.out_features):
            specs.append(TensorSpec(n + ".weight", (o, self.in_features), "matrix"))
            if self.has_bias:
                specs.append(TensorSpec(n + ".bias", (o,), "bias"))
        return specs

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        mats = [get(n + ".weight") for n in self.names]
        self.weight = _to_device(mats, rt.dtype, rt.device)
        self._pack(rt)
        if self.has_bias:
            self.bias = _to_device([get(n + ".bias") for n in self.names], torch.float32, rt.device)

    def matrix_elements(self) -> int:
        return self.in_features * self.total_out

    def bind_shared(self, weight: torch.Tensor, rt: Runtime) -> None:
        """Use a matrix that another part already holds on the device (tied embeddings)."""
        self.rt = rt
        self.weight = weight
        self._pack(rt)

    def _pack(self, rt: Runtime) -> None:
        """The packed copy, if the runtime wants packed weights and its budget still holds this one."""
        self.packed = None
        if not (rt.pack_weights and self.weight.dtype == torch.bfloat16):
            return
        need = K.packed_weight_bytes(self.weight.shape[0], self.weight.shape[1])
        if rt.pack_budget is not None:
            if need > rt.pack_budget:
                return
            rt.pack_budget -= need
        try:
            self.packed = K.pack_weights(self.weight, self.out_features[0] if self.gated else 0)
        except torch.cuda.OutOfMemoryError:
            # no room for this copy after all (memory taken since the budget was worked out): the
            # matrix keeps the row-major kernels, which give the same sums in the same order
            self.packed = None
            if rt.pack_budget is not None:
                rt.pack_budget = 0

    def packed_bytes(self) -> int:
        """Bytes of the packed copy that this product holds beside the matrix (0 without one)."""
        return 0 if self.packed is None else self.packed.data.numel() * self.packed.data.element_size()

    def _packed_rows(self, rows_out: Optional[int]) -> Optional[K.PackedWeight]:
        if self.packed is None or rows_out is None:
            return self.packed
        return self.packed.rows(rows_out)

    def weight_bytes(self) -> int:
        """What a step reads of this product: the matrix once (whichever copy) and the bias."""
        total = self.weight.numel() * self.weight.element_size() if self.weight is not None else 0
        return total + (self.bias.numel() * self.bias.element_size() if self.bias is not None else 0)

    def product(self, a, rows_out: Optional[int] = None, swiglu_input: bool = False,
                f32_ok: bool = False) -> torch.Tensor:
        """a . W^T without the bias, as [M, out] or as float32 partial sums [parts, M, out] for a
        consumer kernel that adds parts (and the bias, `bias_rows`).  With `swiglu_input`, `a` is a
        fused gate/up product (maybe in parts) and W is applied to silu(gate) * up; with `f32_ok`
        the consumer also takes a float32 result.  `a` may be a norm's rows without their scale
        (NormedRows), which the product on the packed copy then applies to its result."""
        if isinstance(a, NormedRows):
            pw = self._packed_rows(rows_out)
            if pw is not None and not pw.gate_rows and not swiglu_input:
                splits, chunk = K.packed_plan(a.x.shape[0], pw.N, pw.K)
                out = K.gemm_packed_unscaled_bf16(a.squares, a.eps, pw, None, torch.float32 if f32_ok else self.rt.dtype,
                                                  splits, chunk)
                if out is not None:
                    return out
            a = a.tensor()
        w = self.weight if rows_out is None else self.weight[:rows_out]
        return K.gemm_product(a, w, self.rt.dtype, swiglu_input=swiglu_input, f32_ok=f32_ok,
                              packed=self._packed_rows(rows_out))

    def add_to(self, a: torch.Tensor, residual: Residual):
        """residual.x += a . W^T + bias in one kernel: for the few rows and the shapes that
        gemm_residual_bf16 serves, and for prompts that the library's product serves (its epilogue adds).
        Returns what the product left for the norm that follows (RowSquares: with that norm's rows without
        their scale if residual.norm has a row weight; empty after the library's product), or None when x
        is untouched and the caller takes the product as a tensor."""
        if not isinstance(a, torch.Tensor) or a.dim() != 2:
            return None
        x = residual.x
        if a.shape[0] > K.SKINNY_MAX_ROWS:
            # prompts: the library's product with the sum in its epilogue, where the library serves anyway
            if self.bias is None and K.gemm_library_add(x, a, self.weight, self.packed):
                return K.RowSquares(None, self.weight.shape[0])
            return None
        if self.packed is None or self.packed.gate_rows:
            return None
        if x.dim() != 2 or x.shape != (a.shape[0], self.packed.N):
            return None
        waves, strips = K.residual_plan(a.shape[0], self.packed.N, self.packed.K)
        if not waves:
            return None
        norm_w = residual.norm.row_weight() if residual.norm is not None else None
        return K.gemm_residual_bf16(x, a, self.packed, self.bias, waves, norm_w, strips)

    def gated_product(self, a) -> Optional[torch.Tensor]:
        """silu(a . gate^T) * (a . up^T) as [M, out] in the runtime's type, made in one kernel from the
        packed copy (up to 64 rows the weight-streaming product, for prompts the tiled one); None where that
        does not apply (no packed copy, float32, row counts at which the library's product and a SwiGLU pass
        are faster)."""
        if self.packed is None or not self.packed.gate_rows:
            return None
        if isinstance(a, NormedRows):
            return K.gemm_packed_unscaled_bf16(a.squares, a.eps, self.packed, None, self.rt.dtype, 1,
                                               K.packed_plan(a.x.shape[0], self.packed.N, self.packed.K)[1])
        if a.dim() != 2:
            return None
        if a.shape[0] > K.SKINNY_MAX_ROWS:
            return K.gemm_tiles_bf16(a, self.packed, None, self.rt.dtype) if K.tiles_serve_gated(a.shape[0], a.shape[1]) else None
        return K.gemm_packed_gated_bf16(a, self.packed, self.rt.dtype, K.packed_plan(a.shape[0], self.packed.N, self.packed.K)[1])

    def bias_rows(self, rows_out: Optional[int] = None) -> Optional[torch.Tensor]:
        return self.bias if (self.bias is None or rows_out is None) else self.bias[:rows_out]

    def forward(self, a: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                rows_out: Optional[int] = None) -> torch.Tensor:
        """a [M, in] -> [M, out]; `rows_out` uses only the first rows of the stacked matrix."""
        w = self.weight if rows_out is None else self.weight[:rows_out]
        b = self.bias if (self.bias is None or rows_out is None) else self.bias[:rows_out]
        return K.gemm(a, w, b, out_dtype or self.rt.dtype, packed=self._packed_rows(rows_out))


def _to_device(parts: List[torch.Tensor], dtype: torch.dtype, device: torch.device) -> torch.Tensor:
    """Stack host tensors by rows into one device tensor of `dtype` without a second host copy."""
    rows = sum(p.shape[0] for p in parts)
    shape = (rows,) + tuple(parts[0].shape[1:])
    out = torch.empty(shape, dtype=dtype, device=device)
    r = 0
    for p in parts:
        out[r:r + p.shape[0]].copy_(p)       # converts on the device side of the copy
        r += p.shape[0]
    return out
