"""Token selection for a batch of logit rows, on the device.

The pipeline is the reference's (Daisi.Llogos/Inference/Sampler.cs:26-85): greedy short cut,
penalties, temperature, top-k, min-p, softmax over candidates, typical-p, top-p, draw."""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..ops import kernels as K
from .params import GenerationParams
from .rng import uniform


class Sampler:
    def __init__(self, params: GenerationParams, stop_tokens: Sequence[int] = ()):
        self.params = params
        self.stop_tokens = tuple(stop_tokens)
        if params.prevent_eos and len(self.stop_tokens) > K.MAX_BANNED:
            raise ValueError(f"prevent_eos can ban at most {K.MAX_BANNED} stop tokens, got {len(self.stop_tokens)}")
        self._fresh_seed = None
        if params.seed is None and params.temperature > 0:
            self._fresh_seed = int(np.random.SeedSequence().generate_state(1)[0])

    def uniforms(self, requests: Sequence[int], indices: Sequence[int]) -> List[float]:
        seed = self.params.seed if self.params.seed is not None else self._fresh_seed
        return [uniform(seed, r, i) for r, i in zip(requests, indices)]

    def sample(self, logits: torch.Tensor, requests: Sequence[int], indices: Sequence[int],
               histories: Optional[Sequence[Sequence[int]]] = None) -> torch.Tensor:
        """int32 token ids [R] for float32 logits [R, V].  requests/indices: which request each
        row belongs to and which of its generated tokens this is (for the random stream);
        histories: each row's prompt + generated tokens (for penalties)."""
        p = self.params
        if p.is_greedy:
            return K.argmax(logits)
        arrays = []
        if p.has_penalties:
            if histories is None:
                raise ValueError("penalties need each row's token history")
            win = [list(h[-p.penalty_count:]) if 0 < p.penalty_count < len(h) else list(h) for h in histories]
            width = max(1, max(len(w) for w in win))
            arr = np.zeros((len(win), width), dtype=np.int32)
            for i, w in enumerate(win):
                arr[i, :len(w)] = w
            arrays = [arr, np.asarray([len(w) for w in win], dtype=np.int32)]
        if p.temperature > 0:
            arrays.append(np.asarray(self.uniforms(requests, indices), dtype=np.float32))
        staged = self._to_device(arrays, logits.device)
        hist, hist_len = (staged[0], staged[1]) if p.has_penalties else (None, None)
        banned = self.stop_tokens if p.prevent_eos else ()
        work = K.sample_prepare(logits, hist, hist_len, p.repetition_penalty, p.frequency_penalty,
                                p.presence_penalty, p.temperature, p.penalize_newline, banned)
        if p.temperature == 0:
            return K.argmax(work)
        return K.sample_pipeline(work, staged[-1], p.top_k, p.top_p, p.min_p, p.typical_p, p.min_keep)

    def _to_device(self, arrays, device) -> List[torch.Tensor]:
        """The step's small host arrays (int32 or float32) on the device with one copy, without
        the host waiting for the work already queued there (a copy from ordinary host memory
        would): through one of a few pinned staging buffers, each free again once its last copy
        has run."""
        if not arrays:
            return []
        n = sum(a.size for a in arrays)
        ring = getattr(self, "_staging", None)
        if ring is None or ring[0][0].numel() < n:
            ring = self._staging = [(torch.empty(max(1024, 2 * n), dtype=torch.int32, pin_memory=True),
                                     torch.cuda.Event()) for _ in range(4)]
            self._staging_next = 0
        host, copied = ring[self._staging_next]
        self._staging_next = (self._staging_next + 1) % len(ring)
        copied.synchronize()
        flat = host.numpy()
        o = 0
        for a in arrays:
            flat[o:o + a.size] = a.reshape(-1).view(np.int32)          # float32 goes as its bits
            o += a.size
        dev = torch.empty(n, dtype=torch.int32, device=device)
        dev.copy_(host[:n], non_blocking=True)
        copied.record()
        out, o = [], 0
        for a in arrays:
            t = dev[o:o + a.size]
            out.append((t.view(torch.float32) if a.dtype == np.float32 else t).view(a.shape))
            o += a.size
        return out
