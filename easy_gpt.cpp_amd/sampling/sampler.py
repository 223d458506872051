"""Sampling of next tokens from float32 logits, on the device.

Options and their meaning are the reference's (/root/reference/src/sampler.cpp:39-105,
defaults from /root/reference/include/cli_options.hpp:9-24): greedy (or temperature <= 0)
takes the first maximum; otherwise probabilities are raised to 1/T (softmax(logits/T)),
cut to the top_k most likely (0 disables), then to the smallest set whose mass reaches
top_p (1 disables), and one uniform number picks a token from what is left.

The reference draws from one shared mt19937 in batch order, so a request's tokens
depend on its neighbours.  Here the uniform number of a request's n-th token is a
function of (seed, request serial, n) alone, so batching changes nothing.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import kernels


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.8
    top_p: float = 0.95
    top_k: int = 20
    greedy: bool = False
    seed: int = 42

    def __post_init__(self):
        if not self.greedy and not self.temperature > 0:
            raise ValueError("Temperature must be greater than 0")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError("Top-p must be in (0, 1]")
        if self.top_k < 0:
            raise ValueError("Top-k must be >= 0")
        if self.seed < 0:
            raise ValueError("Seed must be >= 0")


_MASK = (1 << 64) - 1


def _mix(z: int) -> int:
    """splitmix64 finaliser"""
    z = (z + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform_for(seed: int, serial: int, n: int) -> float:
    """A number in [0, 1) for the n-th token of request `serial` under `seed`."""
    z = _mix(_mix(_mix(seed) ^ serial) ^ n)
    return (z >> 40) / float(1 << 24)


class PendingTokens:
    """Sampled tokens that are still on their way: `device` int32 [R] holds them as soon as the stream gets there
    (the next step can take its token ids from it without the host ever seeing them), `result()` waits for the copy
    to the host that was queued right behind the sampling kernel, and for nothing queued after it."""

    def __init__(self, device: torch.Tensor):
        self.device = device
        self._host = None
        self._event = None
        if device.is_cuda:
            self._host = torch.empty(device.shape, dtype=device.dtype, pin_memory=True)
            self._host.copy_(device, non_blocking=True)
            self._event = torch.cuda.Event()
            self._event.record()

    def result(self) -> list[int]:
        if self._event is None:
            return self.device.tolist()
        self._event.synchronize()
        return self._host.tolist()


class Sampler:
    def __init__(self, device):
        from ..parts.model import resolve_device

        self.device = resolve_device(device)

    def sample(self, logits: torch.Tensor, params: list[SamplingParams], serials: list[int], counts: list[int]) -> list[int]:
        """One token per row of `logits` [R, V]; row r belongs to request serials[r], which has
        produced counts[r] tokens so far."""
        return self.sample_async(logits, params, serials, counts).result()

    def sample_async(self, logits: torch.Tensor, params: list[SamplingParams], serials: list[int],
                     counts: list[int]) -> PendingTokens:
        """The same without waiting for the tokens (`PendingTokens`)."""
        r = logits.shape[0]
        if not (len(params) == len(serials) == len(counts) == r):
            raise ValueError("one SamplingParams, serial and count per row of logits is needed")
        out = torch.empty(r, dtype=torch.int32, device=logits.device)
        k = kernels.backend()
        if all(p.greedy for p in params):
            k.argmax(logits, out)
        else:
            # one row per option, so that each is a contiguous view of one upload; from pinned memory, so that the
            # copy is queued behind the step instead of making the host wait for it (a copy from pageable memory
            # would: with a step launched ahead, that is the step whose tokens are not needed yet)
            pinned = logits.is_cuda
            host = torch.empty((4, r), dtype=torch.float32, pin_memory=pinned)
            rows = host.numpy()
            rows[0] = [0.0 if p.greedy else p.temperature for p in params]
            rows[1] = [p.top_p for p in params]
            rows[2] = [uniform_for(p.seed, s, n) for p, s, n in zip(params, serials, counts)]
            rows[3].view("int32")[:] = [p.top_k for p in params]
            dev = host.to(logits.device, non_blocking=pinned)
            k.sample(logits, dev[0], dev[3].view(torch.int32), dev[1], dev[2], out)
        return PendingTokens(out)
