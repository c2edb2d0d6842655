"""Drawing one token per sequence from float32 logits on the GPU.

The draw of sequence s at its step t uses the uniform number that
Philox4x32-10 gives for key = seed and counter = (t, s, 0, 0): it does not
depend on which other sequences share the batch."""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..kernels import ops
from .config import SamplingConfig


class Drawn:
    """The tokens of one draw: on the device at once (`device`, int32 [B], valid until the
    sampler's next draw has been launched), on the host when `tokens()` is asked for."""

    def __init__(self, device: torch.Tensor, host: torch.Tensor, done: "torch.cuda.Event"):
        self.device, self._host, self._done = device, host, done

    def tokens(self) -> List[int]:
        self._done.synchronize()
        return self._host.tolist()


class Sampler:
    def __init__(self, config: SamplingConfig, device):
        self.config = config
        self.device = device
        self._probs = None
        self._stage = None               # pinned (sequence, step) pairs, and their copy on the device
        self._counters = None
        self._out = None
        self._uploaded = None
        self._host = None                # two pinned buffers for the tokens, used in turn
        self._turn = 0

    def draw(self, logits: torch.Tensor, seq_ids: Sequence[int], steps: Sequence[int]) -> Drawn:
        """logits: float32 [B, V] on the GPU -> B token ids, without waiting for them: the
        kernel and the copy to the host are launched, `Drawn.tokens()` waits."""
        B, V = logits.shape
        c = self.config
        if self._stage is None or self._stage.shape[0] < B:
            cap = max(B, 64)
            self._stage = torch.empty((cap, 2), dtype=torch.int32).pin_memory()
            self._counters = torch.empty((cap, 2), dtype=torch.int32, device=logits.device)
            self._out = torch.empty((cap,), dtype=torch.int32, device=logits.device)
            self._host = [torch.empty((cap,), dtype=torch.int32).pin_memory() for _ in range(2)]
            self._uploaded = None
        if self._uploaded is not None:
            self._uploaded.synchronize()             # the pinned pairs are free to be written again
        stage = self._stage.numpy()
        stage[:B, 0] = seq_ids
        stage[:B, 1] = steps
        counters = self._counters[:B]
        counters.copy_(self._stage[:B], non_blocking=True)
        if self._uploaded is None:
            self._uploaded = torch.cuda.Event()
        self._uploaded.record()
        if self._probs is None or self._probs.shape[0] < B or self._probs.shape[1] != V:
            self._probs = torch.empty((B, V), dtype=torch.float32, device=logits.device)
        out = self._out[:B]
        ops.sample(logits.contiguous(), float(c.temperature), int(c.top_k or 0), float(c.top_p or 0.0),
                   int(c.seed), counters, self._probs[:B], out)
        host = self._host[self._turn][:B]
        self._turn ^= 1
        host.copy_(out, non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        return Drawn(out, host, done)

    def sample(self, logits: torch.Tensor, seq_ids: Sequence[int], steps: Sequence[int]) -> List[int]:
        """logits: float32 [B, V] on the GPU -> B token ids."""
        return self.draw(logits, seq_ids, steps).tokens()

    def last_distribution(self, B: int) -> torch.Tensor:
        """The probabilities the last draw was made from (temperature > 0)."""
        return self._probs[:B]
