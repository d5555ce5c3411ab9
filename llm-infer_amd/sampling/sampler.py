"""Greedy and temperature sampling (tools/infer.cpp:34-106), on the device.

``temperature <= 0`` takes the first maximum; otherwise p = softmax(logits / T) and the
token is the first whose cumulative probability exceeds a uniform number.  The
reference draws that number from one ``mt19937`` for its single sequence
(infer.cpp:36-51, seed 0 = random device); here every sequence has a key and a
counter in the cache's per-sequence state, so its tokens depend on (seed, request
index) only, not on the batch it runs in, and seed 0 is an ordinary fixed seed.
"""
from __future__ import annotations

import torch

from ..kernels import ops

_MASK = (1 << 64) - 1


def request_key(seed: int, request_index: int) -> int:
    """Key of a request's generator, as a signed 64-bit value for an int64 tensor."""
    k = ((seed & _MASK) * 0x9E3779B97F4A7C15 + (request_index & _MASK) * 0xD1B54A32D192ED03 + 1) & _MASK
    return k - (1 << 64) if k >= (1 << 63) else k


class Sampler:
    def __init__(self, temperature: float = 1.0, seed: int = 0):
        self.temperature, self.seed = float(temperature), int(seed)

    def start(self, cache, slots, request_indices) -> None:
        """Set each sequence's generator to the start of its own stream."""
        rows = torch.tensor([[request_key(self.seed, r), 0] for r in request_indices], dtype=torch.int64,
                            device=cache.device)
        idx = torch.tensor(list(slots), dtype=torch.int64, device=cache.device)
        cache.seq_state.index_copy_(0, idx, rows)

    def sample(self, logits: torch.Tensor, seq_slot: torch.Tensor, cache, out=None, temperature_dev=None) -> torch.Tensor:
        """logits float32 [B, V], seq_slot int32 [B] -> token ids int32 [B] on the device.
        ``temperature_dev``: this sampler's (positive) temperature as a float32 on the device, read by
        the kernels instead of the host's value."""
        if self.temperature <= 0.0:
            return ops.argmax(logits, out)
        return ops.sample(logits, self.temperature, seq_slot, cache.seq_state, out=out, temperature_dev=temperature_dev)

    @staticmethod
    def token_prob(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
        """Probability of tokens[r] under softmax(logits[r]) at temperature 1 (infer.cpp:77-81)."""
        return ops.token_prob(logits, tokens)

    def uniform(self, request_index: int, n: int) -> float:
        """The n-th uniform number of a request's stream (host twin of the device generator)."""
        return ops.uniform01(request_key(self.seed, request_index), n)
