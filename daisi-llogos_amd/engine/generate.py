"""The generation loop above the step function: batches of unequal prompts, stop tokens,
sequences that end earlier, and as many batches one after another as there are requests.

One sequence of the loop is the reference's (Daisi.Llogos/Inference/TextGenerator.cs:26-121):
prefill, then sample -> stop check (a sampled stop token ends the sequence and is not
emitted, :78-79) -> emit -> forward, at most MaxTokens times (:73); statistics as :118-120."""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Iterator, List, Optional, Sequence, Tuple

from ..cache.pages import pages_for
from ..sampling.params import GenerationParams


@dataclass
class GenerationResult:
    tokens: List[List[int]]
    finish_reasons: List[str]                 # 'stop' (a stop token was drawn) or 'length'
    prompt_tokens: int = 0
    generated_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_seconds: float = 0.0
    batches: List[List[int]] = field(default_factory=list)

    @property
    def prefill_tokens_per_second(self) -> float:
        return self.prompt_tokens / self.prefill_seconds if self.prefill_seconds > 0 else 0.0

    @property
    def decode_tokens_per_second(self) -> float:
        return self.generated_tokens / self.decode_seconds if self.decode_seconds > 0 else 0.0


def plan_batches(prompt_lens: Sequence[int], max_new_tokens: int, max_batch: int, pool_pages: int) -> List[List[int]]:
    """Requests in their order, cut into batches: at most `max_batch` sequences, and the pages
    all of a batch's sequences can come to hold (prompt + new tokens, rounded up to pages)
    fit the pool.  A request that cannot fit alone is an error."""
    if max_batch <= 0:
        raise ValueError("max_batch must be positive")
    batches: List[List[int]] = []
    cur: List[int] = []
    used = 0
    for i, n in enumerate(prompt_lens):
        if n <= 0:
            raise ValueError(f"request {i} has an empty prompt")
        need = pages_for(n + max_new_tokens)
        if need > pool_pages:
            raise ValueError(f"request {i} needs {need} cache pages ({n} prompt + {max_new_tokens} new tokens), "
                             f"the cache has {pool_pages}")
        if cur and (len(cur) >= max_batch or used + need > pool_pages):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


class Generator:
    """Drives an engine (anything with alloc_slot, free_slot, step and cache.n_pages) and a
    sampler (anything with sample(logits, requests, indices, histories) -> ids)."""

    def __init__(self, engine, max_batch: int = 64, synchronize: Optional[Callable[[], None]] = None,
                 look_ahead: bool = True):
        self.engine = engine
        self.max_batch = max_batch
        self._sync = synchronize or (lambda: None)
        self.look_ahead = look_ahead              # start a step before the host has seen the last one's tokens

    def stop_tokens(self, params: GenerationParams) -> Tuple[int, ...]:
        if params.stop_tokens is not None:
            return tuple(params.stop_tokens)
        spec = getattr(getattr(self.engine, "model", None), "spec", None)
        return tuple(getattr(spec, "eos_token_ids", ()) or ())

    def generate(self, prompts: Sequence[Sequence[int]], params: GenerationParams, sampler=None,
                 on_token: Optional[Callable[[int, int], None]] = None) -> GenerationResult:
        if sampler is None:
            from ..sampling.sampler import Sampler
            sampler = Sampler(params, self.stop_tokens(params))
        stops = set(self.stop_tokens(params))
        prompts = [list(p) for p in prompts]
        result = GenerationResult(tokens=[[] for _ in prompts], finish_reasons=["length"] * len(prompts))
        result.batches = plan_batches([len(p) for p in prompts], params.max_tokens, self.max_batch,
                                      self.engine.cache.n_pages)
        for batch in result.batches:
            self._run_batch(batch, prompts, params, sampler, stops, result, on_token)
        return result

    def _run_batch(self, batch, prompts, params, sampler, stops, result, on_token) -> None:
        eng = self.engine
        slots = {r: eng.alloc_slot() for r in batch}
        try:
            if params.max_tokens == 0:
                return
            if self.look_ahead and getattr(eng, "takes_device_ids", False):
                self._decode_ahead(batch, slots, prompts, params, sampler, stops, result, on_token)
            else:
                self._decode_in_step(batch, slots, prompts, params, sampler, stops, result, on_token)
        finally:
            for r in list(slots):
                eng.free_slot(slots.pop(r))

    def _decode_in_step(self, batch, slots, prompts, params, sampler, stops, result, on_token) -> None:
        """Every step waits for its tokens on the host before the next one starts (engines that
        take their tokens from the host only)."""
        eng = self.engine
        live = list(batch)
        need_history = params.has_penalties
        self._sync()
        t0 = time.perf_counter()
        logits = eng.step([(slots[r], prompts[r]) for r in live], want="last")
        ids = self._sample(sampler, logits, live, prompts, result, need_history)
        t1 = time.perf_counter()
        result.prefill_seconds += t1 - t0
        result.prompt_tokens += sum(len(prompts[r]) for r in live)
        while True:
            nxt = []
            for r, tok in zip(live, ids):
                if self._take_token(r, tok, slots, params, stops, result, on_token):
                    nxt.append((r, tok))
            if not nxt:
                break
            live = [r for r, _ in nxt]
            logits = eng.step([(slots[r], [tok]) for r, tok in nxt], want="last")
            ids = self._sample(sampler, logits, live, prompts, result, need_history)
        self._sync()
        result.decode_seconds += time.perf_counter() - t1

    def _take_token(self, r, tok, slots, params, stops, result, on_token) -> bool:
        """Books request r's next drawn token; False when the request is finished with it (a
        stop token, which is not emitted, or the last token it may have).  A finished request
        gives its slot and pages back at once."""
        if tok in stops:
            result.finish_reasons[r] = "stop"
            self.engine.free_slot(slots.pop(r))
            return False
        result.tokens[r].append(tok)
        result.generated_tokens += 1
        if on_token is not None:
            on_token(r, tok)
        if len(result.tokens[r]) >= params.max_tokens:
            self.engine.free_slot(slots.pop(r))
            return False
        return True

    def _decode_ahead(self, batch, slots, prompts, params, sampler, stops, result, on_token) -> None:
        """The same loop with the host one step behind the device: step t + 1 takes its tokens
        from the device memory that step t's sampler wrote and is started before the host has
        seen them, so the host's work per step (bookkeeping, page tables, the launch) runs while
        the device computes.  The host reads step t's tokens while step t + 1 runs, and only then
        queues step t + 1's sampler, which can so be given every row's tokens up to t (penalties
        look at them).  A request whose token turns out to be a stop token has then run one step
        too many: its result is dropped, and its slot is given back as usual (later work on the
        device comes after that step in stream order).  Requests never take more steps than
        their share of the cache allows: one that has its last permitted token coming is not
        stepped ahead."""
        eng = self.engine
        lend = {"borrow": True} if getattr(eng, "lends_logits", False) else {}
        live = list(batch)
        need_history = params.has_penalties
        history = (lambda rs: [recent_tokens(prompts[r], result.tokens[r], params.penalty_count) for r in rs]) \
            if need_history else (lambda rs: None)
        self._sync()
        t0 = time.perf_counter()
        logits = eng.step([(slots[r], prompts[r]) for r in live], want="last")
        ids = sampler.sample(logits, live, [0] * len(live), history(live))
        # rows: (request, its row in ids); fetch: the tokens on their way to the host
        rows, fetch = [(r, i) for i, r in enumerate(live)], fetch_tokens(ids)
        fetch_first = fetch
        result.prompt_tokens += sum(len(prompts[r]) for r in live)
        t1 = None
        while rows:
            # requests that go on if their pending token is no stop token: step them now
            ahead = [(r, i) for r, i in rows if len(result.tokens[r]) + 1 < params.max_tokens]
            logits = None
            if ahead:
                # (the sampler reads these logits before the next step is queued: they may be the step's own buffer)
                logits = eng.step([(slots[r], [0]) for r, _ in ahead], want="last",
                                  device_ids=(ids, [i for _, i in ahead]), **lend)
            toks = fetch()
            if t1 is None and fetch is fetch_first:                       # the prompt step has ended
                t1 = time.perf_counter()
                result.prefill_seconds += t1 - t0
            went_on = set()
            for r, i in rows:
                if self._take_token(r, int(toks[i]), slots, params, stops, result, on_token):
                    went_on.add(r)
            ids = fetch = None
            if ahead and went_on:
                # (the rows of requests that have just ended are drawn too, and dropped)
                stepped = [r for r, _ in ahead]
                ids = sampler.sample(logits, stepped, [len(result.tokens[r]) for r in stepped], history(stepped))
                fetch = fetch_tokens(ids)
            rows = [(r, j) for j, (r, _) in enumerate(ahead) if r in went_on]
        self._sync()
        result.decode_seconds += time.perf_counter() - (t1 if t1 is not None else t0)

    @staticmethod
    def _sample(sampler, logits, live, prompts, result, need_history) -> List[int]:
        indices = [len(result.tokens[r]) for r in live]
        histories = None
        if need_history:
            count = getattr(sampler, "params", None)
            count = count.penalty_count if count is not None else 0
            histories = [recent_tokens(prompts[r], result.tokens[r], count) for r in live]
        ids = sampler.sample(logits, live, indices, histories)
        return [int(t) for t in (ids.tolist() if hasattr(ids, "tolist") else ids)]


def recent_tokens(prompt: List[int], generated: List[int], count: int) -> List[int]:
    """The last `count` tokens of prompt + generated (all of them for count <= 0) without
    joining the two lists whole at every step."""
    if count <= 0:
        return prompt + generated
    if len(generated) >= count:
        return generated[-count:]
    return prompt[max(0, len(prompt) - (count - len(generated))):] + generated


def fetch_tokens(ids):
    """Starts bringing sampled token ids to the host; the returned function waits for them and
    gives a list.  Device tensors are copied into pinned memory behind the work already queued
    on their stream; anything else (arrays of a stand-in engine) is taken as it is."""
    if hasattr(ids, "is_cuda") and ids.is_cuda:
        import torch
        host = torch.empty(ids.shape, dtype=ids.dtype, pin_memory=True)
        host.copy_(ids, non_blocking=True)
        done = torch.cuda.Event()
        done.record()

        def wait():
            done.synchronize()
            return host.tolist()
        return wait
    return lambda: [int(t) for t in (ids.tolist() if hasattr(ids, "tolist") else ids)]
