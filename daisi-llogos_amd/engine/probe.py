"""Where a step's time goes, kernel group by kernel group, from events on the stream.

The reference's benchmark prints prefill and decode rates (Daisi.Llogos.Cli/Program.cs:292-296,
Daisi.Llogos/Inference/TextGenerator.cs:126-186); it has no per-kernel account.  Here a step can
be run with a probe: the model, its blocks and their parts call `ctx.mark(name)` when the
kernels of a part have been queued, the probe records an event there, and the time between
two marks is the time of the kernels queued between them."""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, List, Tuple

import torch


class StepProbe:
    """Collects marks of one or several steps; `totals()` gives, per name, how many intervals ended at a
    mark of that name and how many milliseconds they took together.

    The host queues a step's kernels more slowly than the GPU runs the short ones, and an interval would
    then hold the GPU's waiting.  `hold(ms)` queues a spin of that length first, so that the host gets
    ahead of the GPU before the first mark."""

    _spin_cycles_per_ms = None          # of the counter that torch.cuda._sleep counts, measured once

    def __init__(self):
        self._marks: List[Tuple[str, torch.cuda.Event]] = []

    def hold(self, milliseconds: float = 20.0) -> None:
        cls = type(self)
        if cls._spin_cycles_per_ms is None:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            a.record()
            torch.cuda._sleep(2_000_000)
            b.record()
            b.synchronize()
            cls._spin_cycles_per_ms = 2_000_000 / max(a.elapsed_time(b), 1e-3)
        torch.cuda._sleep(int(milliseconds * cls._spin_cycles_per_ms))

    def start(self) -> None:
        self("start")

    def context(self, ctx, caches) -> None:
        """The step's context and the layers' views of the cache, as the engine made them: kept for a
        caller that runs single parts of the step again (a record between every two kernels costs
        the short kernels of a single-token step more than they take; see `repeat`)."""
        self.step_context, self.layer_caches = ctx, caches

    def repeat(self, calls) -> float:
        """Microseconds a call of the given functions run one after the other with nothing between them
        (one part of every layer, say: each call then finds its weights in memory, not in a cache)."""
        calls = list(calls)
        before, after = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        self.hold()
        before.record()
        for call in calls:
            call()
        after.record()
        after.synchronize()
        return 1e3 * before.elapsed_time(after) / max(1, len(calls))

    def __call__(self, name: str) -> None:
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self._marks.append((name, ev))

    def totals(self) -> "OrderedDict[str, Tuple[int, float]]":
        torch.cuda.synchronize()
        out: "OrderedDict[str, Tuple[int, float]]" = OrderedDict()
        for (_, before), (name, after) in zip(self._marks, self._marks[1:]):
            if name == "start":
                continue
            n, ms = out.get(name, (0, 0.0))
            out[name] = (n + 1, ms + before.elapsed_time(after))
        return out

    def microseconds_per_call(self) -> Dict[str, float]:
        return {name: 1e3 * ms / n for name, (n, ms) in self.totals().items()}
