"""Weights by tensor name.  The model says which tensors it needs and of which shape; the
checkpoint is compared with that list first, and every difference is reported in one
error: missing tensors, unexpected ones, wrong shapes.

The reference reads by name too and raises on the first missing tensor
(Daisi.Llogos/Model/ModelLoader.cs:140-162); it does not check shapes.  Tensors keep the
element type they are stored in until a part binds them: matrices go to the runtime's
type, norm weights and biases to float32, integer tables to int32."""
from __future__ import annotations

from typing import Callable, Dict, List, Optional

import torch

from ..parts.base import TensorSpec
from .safetensors_io import SafetensorsFile, open_model_files


class WeightError(ValueError):
    """The checkpoint does not fit the model; the message lists every difference."""

    def __init__(self, missing: List[str], unexpected: List[str], wrong_shape: List[str], where: str = ""):
        self.missing, self.unexpected, self.wrong_shape = missing, unexpected, wrong_shape
        lines = [f"checkpoint {where} does not fit the model:".replace("  ", " ")]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        super().__init__("\n".join(lines))


def check_tensors(specs: List[TensorSpec], available: Dict[str, tuple], where: str = "",
                  ignore: Callable[[str], bool] = lambda name: False) -> None:
    """Compare what the model needs with the names and shapes the checkpoint has."""
    wanted = {s.name: s for s in specs}
    missing = [s.name for s in specs if not s.optional and s.name not in available]
    unexpected = sorted(n for n in available if n not in wanted and not ignore(n))
    wrong = [f"{n}: expected {list(wanted[n].shape)}, found {list(available[n])}"
             for n in wanted if n in available and tuple(available[n]) != tuple(wanted[n].shape)]
    if missing or unexpected or wrong:
        raise WeightError(missing, unexpected, wrong, where)


def _ignorable(name: str) -> bool:
    # buffers some exporters store although they are derived from the configuration
    return name.endswith("rotary_emb.inv_freq")


class Checkpoint:
    """The tensors of a model folder, by name."""

    def __init__(self, folder: str):
        self.folder = folder
        self.files: List[SafetensorsFile] = open_model_files(folder)
        self.where: Dict[str, SafetensorsFile] = {}
        for f in self.files:
            for n in f.names:
                self.where[n] = f

    def shapes(self) -> Dict[str, tuple]:
        return {n: f.shape(n) for n, f in self.where.items()}

    def get(self, name: str) -> Optional[torch.Tensor]:
        f = self.where.get(name)
        if f is None:
            return None
        t = f.tensor(name)
        if not t.dtype.is_floating_point:
            t = t.to(torch.int32)
        return t

    def check(self, specs: List[TensorSpec], tied_head: Optional[str] = None) -> None:
        def ignore(name: str) -> bool:
            # a tied model may still store its head; it equals the embedding and is not read
            return _ignorable(name) or (tied_head is not None and name == tied_head)
        check_tensors(specs, self.shapes(), f"'{self.folder}'", ignore)

    def close(self) -> None:
        for f in self.files:
            f.close()
