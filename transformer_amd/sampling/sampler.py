"""Chooses next tokens on the GPU from float32 logits.

The reference draws one unseeded random number per logits row and hands it to
its sampling operator together with (temperature, top_p, top_k)
(tensor/src/operators/random_sample.rs:64-75). Here the number
comes from a counter-based generator keyed by (seed, sequence number, tokens
generated so far), so a sequence draws the same numbers whatever batch it is in
and a run can be repeated.
"""
from __future__ import annotations

from typing import Sequence

import numpy as np
import torch

from .. import kernels
from .args import SampleArgs

_M64 = (1 << 64) - 1


def uniform(seed: int, sequence: int, drawn: int) -> float:
    """u in [0, 1) with 24 random bits: a splitmix64 finaliser over the three keys."""
    z = (seed * 0x9E3779B97F4A7C15 + sequence * 0xBF58476D1CE4E5B9
         + drawn * 0x94D049BB133111EB + 0x2545F4914F6CDD1D) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    z ^= z >> 31
    return (z >> 40) / float(1 << 24)


class Chosen:
    """Tokens that the GPU has been asked to choose: ``device`` holds them (int32) as soon as
    the stream gets there; ``result()`` waits for their copy to the host."""

    def __init__(self, device: torch.Tensor, host: torch.Tensor, event):
        self.device, self._host, self._event = device, host, event

    def result(self):
        self._event.synchronize()
        return self._host.tolist()


class Sampler:
    RING = 4        # choices that may be outstanding before a buffer is used again

    def __init__(self, args: SampleArgs = SampleArgs(), seed: int = 0, device="cuda:0"):
        self.args, self.seed, self.device = args, int(seed), torch.device(device)
        self._ring = [None] * self.RING
        self._turn = 0

    def _buffers(self, n: int):
        i = self._turn
        self._turn = (i + 1) % self.RING
        b = self._ring[i]
        if b is None or b[0].numel() < n:
            cap = max(64, n)
            b = (torch.empty(cap, dtype=torch.int32, device=self.device),
                 torch.empty(cap, dtype=torch.float32, device=self.device),
                 torch.empty(cap, dtype=torch.float32, pin_memory=True),
                 torch.empty(cap, dtype=torch.int32, pin_memory=True))
            self._ring[i] = b
        return b[0][:n], b[1][:n], b[2][:n], b[3][:n]

    def choose_async(self, logits: torch.Tensor, sequences: Sequence[int], drawn: Sequence[int]) -> Chosen:
        """logits: float32 [n, vocab] on the GPU. sequences[i], drawn[i]: the keys of
        row i's random number. Nothing here waits for the GPU."""
        n = logits.shape[0]
        out, u_dev, u_host, out_host = self._buffers(n)
        if self.args.greedy:
            kernels.argmax(logits, out)
        else:
            u_host.numpy()[:] = np.asarray([uniform(self.seed, s, d) for s, d in
                                            zip(sequences, drawn)], dtype=np.float32)
            u_dev.copy_(u_host, non_blocking=True)
            k = self.args.top_k if self.args.top_k is not None else logits.shape[1]
            kernels.sample(logits, u_dev, out, float(self.args.temperature), int(k),
                           float(self.args.top_p))
        out_host.copy_(out, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        return Chosen(out, out_host, ev)

    def choose(self, logits: torch.Tensor, sequences: Sequence[int], drawn: Sequence[int]):
        """As ``choose_async``, returning the chosen tokens as a list of ints."""
        return self.choose_async(logits, sequences, drawn).result()
