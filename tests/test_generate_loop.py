"""The generation loop's decisions, with a model of straw (no GPU): stop ids,
sequences that end earlier, batches one after another, slots used again."""
from typing import List

import pytest
import torch

from torchless_rs_amd.engine.generate import generate, plan_batches

V = 50


class StrawEngine:
    """Next token = (last token + 1) mod V.  Keeps books like the real one."""

    def __init__(self, slots=4, pages=64):
        self.free_slots = list(range(slots - 1, -1, -1))
        self.held = {}
        self.pages = pages
        self.steps: List[List[int]] = []          # lengths of each step's entries
        self.alloc_log: List[int] = []

    def alloc(self):
        s = self.free_slots.pop()
        self.held[s] = []
        self.alloc_log.append(s)
        return s

    def free(self, s):
        assert s in self.held, "freed twice"
        del self.held[s]
        self.free_slots.append(s)

    def fits(self, lengths):
        return len(lengths) <= len(self.free_slots) and sum(-(-n // 64) for n in lengths) <= self.pages

    def step(self, batch):
        self.steps.append([len(b.tokens) for b in batch])
        out = torch.zeros(len(batch), V)
        for i, b in enumerate(batch):
            assert b.slot in self.held and list(b.want) == [len(b.tokens) - 1]
            self.held[b.slot] += list(b.tokens)
            out[i, (self.held[b.slot][-1] + 1) % V] = 1.0
        return out


class ArgmaxSampler:
    def __init__(self):
        self.calls = []

    def sample(self, logits, seq_ids, steps):
        self.calls.append((list(seq_ids), list(steps)))
        return logits.argmax(-1).tolist()


def test_counts_and_order():
    eng, smp = StrawEngine(), ArgmaxSampler()
    out = generate(eng, smp, [[1, 2, 3], [10], [20, 21]], max_tokens=4)
    assert [r.tokens for r in out] == [[4, 5, 6, 7], [11, 12, 13, 14], [22, 23, 24, 25]]
    assert all(r.finish_reason == "length" and not r.stopped_at_eos for r in out)
    assert eng.steps == [[3, 1, 2], [1, 1, 1], [1, 1, 1], [1, 1, 1]]     # prompts whole, then one each
    assert not eng.held                                                   # every slot given back
    assert smp.calls[1] == ([0, 1, 2], [1, 1, 1])                         # (request, its step) feed the draw


def test_stop_id_ends_one_sequence_only():
    eng, smp = StrawEngine(), ArgmaxSampler()
    seen = []
    out = generate(eng, smp, [[1], [40], [7]], max_tokens=6, stop_ids=[43, 9],
                   on_token=lambda i, t: seen.append((i, t)))
    assert out[0].tokens == [2, 3, 4, 5, 6, 7] and out[0].finish_reason == "length"
    assert out[1].tokens == [41, 42] and out[1].stopped_at_eos           # 43 is not part of the output
    assert out[2].tokens == [8] and out[2].finish_reason == "stop"
    assert eng.steps == [[1, 1, 1], [1, 1, 1], [1, 1], [1], [1], [1]]     # the batch shrinks
    assert (1, 43) not in seen and (1, 42) in seen and len(seen) == 9
    assert not eng.held


def test_stop_at_first_token_and_zero_budget():
    eng, smp = StrawEngine(), ArgmaxSampler()
    out = generate(eng, smp, [[4]], max_tokens=3, stop_ids=[5])
    assert out[0].tokens == [] and out[0].stopped_at_eos
    out = generate(eng, smp, [[4]], max_tokens=0)
    assert out[0].tokens == [] and out[0].finish_reason == "length" and eng.steps == [[1]]
    with pytest.raises(ValueError, match="empty"):
        generate(eng, smp, [[1], []], max_tokens=2)


def test_batches_one_after_another_reuse_slots():
    eng, smp = StrawEngine(slots=2), ArgmaxSampler()
    prompts = [[i] for i in range(5)]
    out = generate(eng, smp, prompts, max_tokens=2)
    assert [r.tokens for r in out] == [[i + 1, i + 2] for i in range(5)]
    assert [len(s) for s in eng.steps] == [2, 2, 2, 2, 1, 1]              # batches of 2, 2, 1
    assert len(eng.alloc_log) == 5 and set(eng.alloc_log) == {0, 1}       # the same slots again
    out = generate(StrawEngine(slots=4), smp, prompts, max_tokens=1, max_batch=3)
    assert [r.tokens for r in out] == [[i + 1] for i in range(5)]


def test_plan_by_pages():
    fits = lambda ls: sum(-(-n // 64) for n in ls) <= 4
    assert plan_batches([64, 64, 128, 65, 200, 10], fits, None) == [[0, 1, 2], [3], [4], [5]] or \
        plan_batches([64, 64, 128, 65, 200, 10], fits, None) == [[0, 1, 2], [3], [4, 5]]
    assert plan_batches([1] * 5, fits, 2) == [[0, 1], [2, 3], [4]]
    with pytest.raises(ValueError, match="more than the cache holds"):
        plan_batches([10, 300], fits, None)


# ---- running ahead: the next step is launched before the host has read the tokens -----------

class AheadEngine(StrawEngine):
    """Takes a step's tokens from a tensor 'on the device' when asked to."""

    def step(self, batch, device_tokens=None, token_rows=None):
        if device_tokens is not None:
            assert all(list(b.tokens) == [0] for b in batch) and len(token_rows) == len(batch)
            batch = [type(b)(b.slot, [int(device_tokens[r])], b.want) for b, r in zip(batch, token_rows)]
        return super().step(batch)


class DrawingSampler(ArgmaxSampler):
    def __init__(self):
        super().__init__()
        self.unread = 0                # draws whose tokens the host has not looked at yet

    def draw(self, logits, seq_ids, steps):
        self.calls.append((list(seq_ids), list(steps)))
        ids = logits.argmax(-1).to(torch.int32)
        self.unread += 1
        outer = self

        class Drawn:
            device = ids

            def tokens(self):
                outer.unread -= 1
                return ids.tolist()
        return Drawn()


@pytest.mark.parametrize("prompts,max_tokens,stops", [
    ([[1, 2, 3], [10], [20, 21]], 4, []),
    ([[1], [40], [7]], 6, [43, 9]),
    ([[4]], 3, [5]),
    ([[4], [6]], 1, []),
    ([[i] for i in range(5)], 3, [3, 6]),
])
def test_running_ahead_gives_the_same_tokens(prompts, max_tokens, stops):
    seen_a, seen_b = [], []
    a = generate(StrawEngine(slots=2), ArgmaxSampler(), prompts, max_tokens, stops, max_batch=2,
                 on_token=lambda i, t: seen_a.append((i, t)))
    eng, smp = AheadEngine(slots=2), DrawingSampler()
    b = generate(eng, smp, prompts, max_tokens, stops, max_batch=2, on_token=lambda i, t: seen_b.append((i, t)))
    assert [(r.tokens, r.finish_reason) for r in a] == [(r.tokens, r.finish_reason) for r in b]
    assert sorted(seen_a) == sorted(seen_b)
    assert not eng.held and smp.unread == 0                  # every slot given back, every draw read


def test_running_ahead_steps():
    eng, smp = AheadEngine(), DrawingSampler()
    out = generate(eng, smp, [[1], [40], [7]], max_tokens=6, stop_ids=[43, 9])
    assert out[1].tokens == [41, 42] and out[2].tokens == [8]
    # a sequence that draws a stop id has run one row more than without running ahead
    # ([[1, 1, 1], [1, 1, 1], [1, 1], [1], [1], [1]]); budgets are known beforehand: no row past them
    assert eng.steps == [[1, 1, 1], [1, 1, 1], [1, 1, 1], [1, 1], [1], [1]]
    assert smp.calls[2] == ([0, 1, 2], [2, 2, 2])            # (request, its step) as without running ahead
    eng, smp = AheadEngine(), DrawingSampler()
    generate(eng, smp, [[1, 2], [5]], max_tokens=3)
    assert eng.steps == [[2, 1], [1, 1], [1, 1]]             # 3 tokens each: the last is never fed
    out = generate(AheadEngine(), DrawingSampler(), [[1]], max_tokens=5, run_ahead=False)
    assert out[0].tokens == [2, 3, 4, 5, 6]


@pytest.mark.parametrize("fail_at", [0, 3])
def test_an_exception_leaves_nothing_held(fail_at):
    """`on_token` (or a step) that raises: the batch's slots are given back, and the engine serves
    the next call as if nothing had happened."""
    eng, smp = StrawEngine(), ArgmaxSampler()
    seen = []

    def on_token(i, t):
        seen.append((i, t))
        if len(seen) > fail_at:
            raise RuntimeError("the caller's callback failed")

    with pytest.raises(RuntimeError, match="callback failed"):
        generate(eng, smp, [[1, 2], [10], [20]], max_tokens=5, on_token=on_token)
    assert not eng.held and sorted(eng.free_slots) == [0, 1, 2, 3]
    out = generate(eng, smp, [[1, 2], [10]], max_tokens=2)
    assert [r.tokens for r in out] == [[3, 4], [11, 12]] and not eng.held


def test_a_failing_step_leaves_nothing_held():
    class Failing(StrawEngine):
        def step(self, batch):
            if len(self.steps) == 2:
                raise ValueError("no room")
            return super().step(batch)

    eng = Failing()
    with pytest.raises(ValueError, match="no room"):
        generate(eng, ArgmaxSampler(), [[1], [5, 6]], max_tokens=6)
    assert not eng.held
