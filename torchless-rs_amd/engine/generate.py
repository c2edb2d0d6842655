"""The generation loop above the step function.

Per sequence it behaves as the reference's `generate_until_eos`
(src/sampler/mod.rs:269-305): feed the prompt, sample, and go on one token at
a time until `max_tokens` tokens are out or a stop id is drawn; the stop id is
not part of the output and is not counted.  (The reference's single-shot
command line passes no stop ids and always runs `max_tokens`,
src/main.rs:581-597.)  Above that, ours: requests are served in batches of
unequal prompts that start together; a sequence that ends leaves the batch
and gives its slot back while the others go on; when a batch is done the next
requests take the freed slots, until every request is served.

The loop touches the engine only through `alloc`, `free`, `step` and
`fits`, and the sampler through `sample` (or `draw`), so its decisions can be
tested without a GPU.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence

from .engine import SeqInput


@dataclass
class GenerationResult:
    tokens: List[int] = field(default_factory=list)
    finish_reason: str = ""            # "stop" (a stop id was drawn) or "length" (max_tokens reached)

    @property
    def stopped_at_eos(self) -> bool:
        return self.finish_reason == "stop"


def plan_batches(n_tokens_needed: Sequence[int], fits: Callable[[List[int]], bool],
                 max_batch: Optional[int]) -> List[List[int]]:
    """Cut the requests, in their order, into batches: a batch takes requests
    while it stays within `max_batch` and `fits` says that the cache holds
    them all at their full lengths."""
    batches: List[List[int]] = []
    cur: List[int] = []
    for i, need in enumerate(n_tokens_needed):
        trial = cur + [i]
        if cur and ((max_batch and len(trial) > max_batch) or
                    not fits([n_tokens_needed[j] for j in trial])):
            batches.append(cur)
            cur = [i]
        else:
            cur = trial
        if len(cur) == 1 and not fits([need]):
            raise ValueError(f"request {i} needs {need} positions, more than the cache holds; "
                             "raise max_tokens of the engine")
    if cur:
        batches.append(cur)
    return batches


def generate(engine, sampler, prompts: Sequence[Sequence[int]], max_tokens: int,
             stop_ids: Sequence[int] = (), max_batch: Optional[int] = None,
             on_token: Optional[Callable[[int, int], None]] = None,
             run_ahead: Optional[bool] = None) -> List[GenerationResult]:
    """Generate for every prompt; results come back in the order of the
    prompts.  `on_token(request, token)` is called for each token as it is
    produced.

    `run_ahead` (default: if the sampler can `draw`): the next step is launched
    with the drawn tokens still on the device, before the host has read them, so
    that the GPU does not wait while the host looks at tokens and prepares a
    step.  A sequence whose token turns out to be a stop id has then run one
    row too many; the row is dropped with the sequence.  The tokens are the
    same either way."""
    for i, p in enumerate(prompts):
        if len(p) < 1:
            raise ValueError(f"prompt {i} is empty; a prompt needs at least one token")
    stop = set(int(s) for s in stop_ids)
    results = [GenerationResult() for _ in prompts]
    if max_tokens <= 0:
        for r in results:
            r.finish_reason = "length"
        return results
    if run_ahead is None:
        run_ahead = hasattr(sampler, "draw")
    need = [len(p) + max_tokens - 1 for p in prompts]        # the last token is never fed

    def accept(i: int, t: int) -> bool:
        """Book request i's token; is the request finished?"""
        r = results[i]
        if t in stop:
            r.finish_reason = "stop"
        else:
            r.tokens.append(t)
            if on_token is not None:
                on_token(i, t)
            if len(r.tokens) >= max_tokens:
                r.finish_reason = "length"
        return bool(r.finish_reason)

    for batch in plan_batches(need, engine.fits, max_batch):
        run = BatchRun(engine, sampler, accept, max_tokens, run_ahead)
        try:
            run.start(batch, [prompts[i] for i in batch], [len(results[i].tokens) for i in batch])
            while run.advance():
                pass
        finally:
            # whatever ended the batch (a step that failed, the caller's `on_token`, an interrupt),
            # nothing of it stays held in the engine
            run.release()
    return results


class BatchRun:
    """One batch from its prompts to its last token, a step at a time: `start`, then `advance`
    until it returns False.  `accept(request, token) -> finished` books a token for the caller;
    `release` frees what is still held (call it in a `finally`).  `generate` is a loop around
    this, and so is a measurement of decode steps: there is no second decode loop."""

    def __init__(self, engine, sampler, accept: Callable[[int, int], bool], max_tokens: int, run_ahead: bool):
        self.engine, self.sampler, self.accept = engine, sampler, accept
        self.max_tokens, self.run_ahead = max_tokens, run_ahead
        self.slots: Dict[int, int] = {}             # request -> slot, while it is alive
        self.count: Dict[int, int] = {}             # request -> tokens booked so far
        self.order: List[int] = []                  # run ahead: requests whose tokens `drawn` holds, row by row
        self.drawn = None
        self.logits = None                          # not running ahead: what the last step returned
        self.live: List[int] = []

    def start(self, requests: Sequence[int], prompts: Sequence[Sequence[int]], booked: Optional[Sequence[int]] = None) -> None:
        """Take a slot for every request and run all prompts as one step."""
        for i in requests:
            self.slots[i] = self.engine.alloc()
        logits = self.engine.step([SeqInput(self.slots[i], list(p), [len(p) - 1]) for i, p in zip(requests, prompts)])
        self.resume(requests, logits, booked)

    def resume(self, requests: Sequence[int], logits, booked: Optional[Sequence[int]] = None,
               slots: Optional[Sequence[int]] = None) -> None:
        """Go on from `logits`, one row for each request in order, that a caller's own steps
        produced (its prompts fed in pieces, say); `slots`: the requests' slots, if the caller
        took them."""
        if slots is not None:
            self.slots.update(zip(requests, slots))
        self.count = {i: (booked[k] if booked is not None else 0) for k, i in enumerate(requests)}
        self.live = list(requests)
        if self.run_ahead:
            self.order = list(requests)
            self.drawn = self.sampler.draw(logits, self.order, [self.count[i] for i in self.order])
        else:
            self.logits = logits

    def _book(self, i: int, t: int) -> None:
        self.count[i] += 1
        if self.accept(i, t):
            self.engine.free(self.slots.pop(i))

    def advance(self) -> bool:
        """One more step of the batch; False when every request has finished."""
        engine, slots = self.engine, self.slots
        if not self.run_ahead:
            if not self.live:
                return False
            ids = self.sampler.sample(self.logits, self.live, [self.count[i] for i in self.live])
            feed = {}
            for i, t in zip(self.live, ids):
                self._book(i, t)
                if i in slots:
                    feed[i] = [t]
            self.live = [i for i in self.live if i in slots]
            if not self.live:
                return False
            self.logits = engine.step([SeqInput(slots[i], feed[i], [0]) for i in self.live])
            return True
        # run ahead: those of `order` that are not known to be finished go into the next step at once
        order, drawn = self.order, self.drawn
        if not order:
            return False
        # a request that is alive and whose budget this token does not use up goes on, unless
        # the token is a stop id, which the host does not know yet
        rows, ahead = [], []
        for row, i in enumerate(order):
            if i in slots and self.count[i] + 1 < self.max_tokens:
                rows.append(row)
                ahead.append(i)
        nxt_drawn = None
        if ahead:
            logits = engine.step([SeqInput(slots[i], [0], [0]) for i in ahead],
                                 device_tokens=drawn.device, token_rows=rows)
            nxt_drawn = self.sampler.draw(logits, ahead, [self.count[i] + 1 for i in ahead])
        for i, t in zip(order, drawn.tokens()):
            if i in slots:                            # (a request dropped earlier: its row ran for nothing)
                self._book(i, t)
        self.order, self.drawn = ahead, nxt_drawn
        return bool(ahead)

    def release(self) -> None:
        for i in list(self.slots):
            self.engine.free(self.slots.pop(i))
