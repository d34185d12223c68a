"""The generation loop above the step function.

The reference's loop serves one sequence: the whole prompt in the first call,
then the token just produced; the position advances by the tokens fed; a token
equal to the stop token ends the loop and is not emitted; ``max_steps`` bounds
the number of calls (test-utils/src/lib.rs:147-173). Its timing
table counts the first call as prefill and the rest as decode (:159-163,
:175-190).

Here the same rules run for many requests: they are cut into batches that fit
the cache; a batch's prompts, of unequal lengths, go through one step; then
every unfinished sequence of the batch gets one token per step; a sequence that
stops leaves the batch and gives its slot back; the next batch starts when the
batch is empty, in slots that were used before.

The decisions live in ``run_batches`` and need only a *stepper* (alloc, free,
step), so they are tested without a GPU.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

from ..kernels import PAGE   # tokens per cache page: one constant, checked against the kernel library


class GenerationError(ValueError):
    pass


@dataclass
class Timing:
    prefill_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_tokens: int = 0
    decode_seconds: float = 0.0
    decode_steps: int = 0

    def table(self) -> List[Dict[str, object]]:
        """Rows total / prefill / decode with the reference's columns."""
        def row(name, n, s):
            return {"": name, "num tokens": n, "elapse": s,
                    "time per token": (s / n) if n else 0.0,
                    "tokens per second": (n / s) if s > 0 else 0.0}
        return [row("total", self.prefill_tokens + self.decode_tokens,
                    self.prefill_seconds + self.decode_seconds),
                row("prefill", self.prefill_tokens, self.prefill_seconds),
                row("decode", self.decode_tokens, self.decode_seconds)]


@dataclass
class GenerationResult:
    tokens: List[List[int]]                       # generated tokens per request, input order
    finish: List[str]                             # "stop" | "length" per request
    timing: Timing = field(default_factory=Timing)
    batches: List[List[int]] = field(default_factory=list)   # request indices of each batch


def plan_batches(prompt_lens: Sequence[int], max_new_tokens: int, capacity_tokens: int,
                 max_batch: int) -> List[List[int]]:
    """Cuts the requests, in order, into batches whose sequences fit the cache
    together when each grows to prompt + max_new_tokens (rounded up to pages)."""
    if max_batch < 1:
        raise GenerationError("max_batch must be at least 1")
    batches, cur, used = [], [], 0
    for i, n in enumerate(prompt_lens):
        if n < 1:
            raise GenerationError(f"request {i}: a prompt needs at least one token")
        # the last generated token is never fed back, so it needs no cache row
        need = -(-(n + max(max_new_tokens - 1, 0)) // PAGE) * PAGE
        if need > capacity_tokens:
            raise GenerationError(f"request {i}: {n} prompt tokens + {max_new_tokens} new ones need "
                                  f"{need} cache tokens, the cache holds {capacity_tokens}")
        if cur and (used + need > capacity_tokens or len(cur) >= max_batch):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


def run_batches(stepper, prompts: Sequence[Sequence[int]], max_new_tokens: int,
                stop_ids=(), capacity_tokens: int = 1 << 62, max_batch: int = 1 << 30,
                on_token: Optional[Callable[[int, int], None]] = None,
                clock: Callable[[], float] = time.perf_counter,
                max_position: Optional[int] = None) -> GenerationResult:
    """stepper.alloc() -> handle; stepper.free(handle);
    stepper.step([(handle, request index, tokens generated so far, tokens to feed)])
    -> one next token per item (the stepper samples).

    A stepper that also has ``step_async(items, previous, take) -> pending`` is driven one
    step ahead: the next step is started before the tokens of the last one have reached
    the host, taking them from where the last step left them (``previous`` is the last
    step's pending, ``take[j]`` the place of item j in it; the items then carry None for
    their tokens) and ``pending.result()`` gives the tokens later. A sequence that turns
    out to have stopped has then been stepped once more than needed; that step's token is
    dropped. Only the prompts' step is read before the next one starts.

    max_position: positions a sequence may use (the model's context length). A prompt
    longer than that is refused; a sequence that reaches it ends with "length" (its last
    token is never fed back, so a prompt of n tokens can still produce max_position - n + 1)."""
    stop = set(int(s) for s in stop_ids)
    n_req = len(prompts)
    limit = [max_new_tokens] * n_req
    if max_position is not None:
        for i, p in enumerate(prompts):
            if len(p) > max_position:
                raise GenerationError(f"request {i}: a prompt of {len(p)} tokens is longer than the "
                                      f"model's {max_position} positions")
            limit[i] = min(max_new_tokens, max_position - len(p) + 1)
    result = GenerationResult(tokens=[[] for _ in range(n_req)], finish=["length"] * n_req)
    if max_new_tokens <= 0 or n_req == 0:
        return result
    result.batches = plan_batches([len(p) for p in prompts], max_new_tokens, capacity_tokens,
                                  max_batch)
    ahead = hasattr(stepper, "step_async")
    t = result.timing
    for batch in result.batches:
        handles = {i: stepper.alloc() for i in batch}
        live = list(batch)                         # not known to have ended
        feed = {i: list(prompts[i]) for i in batch}
        started = {i: 0 for i in batch}            # steps started for the sequence
        flying = None                              # (pending or tokens, request indices)
        first, t0 = True, clock()

        def settle(tokens, order):
            """The decisions for one step's tokens."""
            nonlocal live
            for i, tok in zip(order, tokens):
                if i not in handles:               # it had ended before this step came back
                    continue
                tok = int(tok)
                if tok in stop:                    # the stop token is not emitted
                    result.finish[i] = "stop"
                else:
                    result.tokens[i].append(tok)
                    if on_token is not None:
                        on_token(i, tok)
                    if len(result.tokens[i]) < limit[i]:
                        feed[i] = [tok]
                        continue
                stepper.free(handles.pop(i))       # the sequence leaves the batch
                live = [x for x in live if x != i]

        def clocked(fed, was_first):
            nonlocal t0
            now = clock()
            if was_first:
                t.prefill_tokens += fed
                t.prefill_seconds += now - t0
            else:
                t.decode_tokens += fed
                t.decode_seconds += now - t0
                t.decode_steps += 1
            t0 = now

        try:
            while True:
                if flying is not None and flying[3]:
                    # the prompts' step is read before the first single-token step starts: the
                    # table's prefill row is then the time to the first token (the reference's
                    # first call, test-utils/src/lib.rs:159-163), whatever the first
                    # single-token step costs (it may be recorded), and a sequence that stops
                    # with its first token is not stepped again
                    settle(flying[0].result(), flying[1])
                    clocked(flying[2], flying[3])
                    flying = None
                run = [i for i in live if started[i] < limit[i]]
                new = None
                if run:
                    if not ahead:
                        items = [(handles[i], i, started[i], feed[i]) for i in run]
                        new = (stepper.step(items), run, sum(len(feed[i]) for i in run), first)
                    elif flying is None:
                        items = [(handles[i], i, started[i], feed[i]) for i in run]
                        new = (stepper.step_async(items, None, None), run,
                               sum(len(feed[i]) for i in run), first)
                    else:
                        items = [(handles[i], i, started[i], None) for i in run]
                        take = [flying[1].index(i) for i in run]
                        new = (stepper.step_async(items, flying[0], take), run, len(run), first)
                    first = False
                    for i in run:
                        started[i] += 1
                if flying is not None:
                    settle(flying[0].result(), flying[1])
                    clocked(flying[2], flying[3])
                    flying = None
                if new is None:
                    break
                if ahead:
                    flying = new
                else:
                    settle(new[0], new[1])
                    clocked(new[2], new[3])
        finally:
            for h in handles.values():
                stepper.free(h)
    return result


class ModelStepper:
    """The stepper over a real model: slots of its cache, its step, a sampler."""

    def __init__(self, model, cache, sampler):
        self.model, self.cache, self.sampler = model, cache, sampler

    def alloc(self):
        return self.cache.alloc_slot()

    def free(self, slot):
        self.cache.free_slot(slot)

    def step_async(self, items, previous=None, take=None):
        """Starts a step and the choice of its tokens; nothing waits for the GPU. With
        ``previous`` the tokens are taken on the GPU from that earlier choice."""
        import torch
        from .batch import Entry
        entries = [Entry(slot, toks if toks is not None else (0,),
                         ((len(toks) if toks is not None else 1) - 1,)) for slot, _, _, toks in items]
        dev = None
        if previous is not None:
            dev = previous.device
            if list(take) != list(range(dev.numel())):
                dev = dev[torch.tensor(list(take), dtype=torch.long, device=dev.device)]
        logits = self.model.step(self.cache, entries, device_tokens=dev)
        return self.sampler.choose_async(logits, [i for _, i, _, _ in items],
                                         [g for _, _, g, _ in items])

    def step(self, items):
        return self.step_async(items).result()


def generate(model, prompts: Sequence[Sequence[int]], max_new_tokens: int, sample_args=None,
             stop_ids=None, seed: int = 0, cache=None, max_batch: Optional[int] = None,
             on_token=None) -> GenerationResult:
    """Generates for every prompt (lists of token ids). ``stop_ids`` defaults to
    the configuration's end-of-sequence ids; ``cache`` to one sized for the
    largest batch this call needs."""
    from ..sampling.args import SampleArgs
    from ..sampling.sampler import Sampler
    sample_args = sample_args or SampleArgs()
    if stop_ids is None:
        stop_ids = model.spec.stop_ids
    max_batch = max_batch or 64
    if cache is None:
        need = sorted((-(-(len(p) + max_new_tokens) // PAGE) * PAGE for p in prompts), reverse=True)
        cache = model.new_cache(max(PAGE, sum(need[:max_batch])), max_slots=max_batch)
    capacity = cache.num_pages * PAGE
    stepper = ModelStepper(model, cache, Sampler(sample_args, seed, model.device))
    return run_batches(stepper, prompts, max_new_tokens, stop_ids, capacity,
                       min(max_batch, cache.max_slots), on_token,
                       max_position=model.spec.max_position)
