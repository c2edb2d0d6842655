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
`fits`, and the sampler through `sample`, so its decisions can be tested
without a GPU.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

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
             on_token: Optional[Callable[[int, int], None]] = None) -> List[GenerationResult]:
    """Generate for every prompt; results come back in the order of the
    prompts.  `on_token(request, token)` is called for each token as it is
    produced."""
    for i, p in enumerate(prompts):
        if len(p) < 1:
            raise ValueError(f"prompt {i} is empty; a prompt needs at least one token")
    stop = set(int(s) for s in stop_ids)
    results = [GenerationResult() for _ in prompts]
    if max_tokens <= 0:
        for r in results:
            r.finish_reason = "length"
        return results
    need = [len(p) + max_tokens - 1 for p in prompts]        # the last token is never fed
    for batch in plan_batches(need, engine.fits, max_batch):
        slots = {i: engine.alloc() for i in batch}
        live = list(batch)
        feed = {i: list(prompts[i]) for i in batch}
        while live:
            logits = engine.step([SeqInput(slots[i], feed[i], [len(feed[i]) - 1]) for i in live])
            ids = sampler.sample(logits, live, [len(results[i].tokens) for i in live])
            nxt = []
            for i, t in zip(live, ids):
                r = results[i]
                if t in stop:
                    r.finish_reason = "stop"
                else:
                    r.tokens.append(t)
                    if on_token is not None:
                        on_token(i, t)
                    if len(r.tokens) >= max_tokens:
                        r.finish_reason = "length"
                if r.finish_reason:
                    engine.free(slots.pop(i))
                else:
                    feed[i] = [t]
                    nxt.append(i)
            live = nxt
    return results
