"""Choosing next tokens from logits: greedy, and temperature / top-k sampling with the
reference's law (generate.py:40-57).

``logits / max(temperature, 1e-5)``, entries below the k-th largest dropped, softmax,
then ``argmax(p / q)`` with ``q ~ Exp(1)`` - a draw from ``p`` that needs no prefix sums
and no host synchronisation.  ``temperature == 0`` is an exact argmax (lowest index on
ties).  The noise is a counter-based function of (seed, request key, position), so a
request's tokens do not depend on what else is in the batch: ``q_i = -log((n_i + 1/2) /
2^23)`` with ``n_i`` the upper 23 bits of word ``i % 4`` of Philox4x32-10 at counter
``(i // 4, position of the token being drawn, request key, 0)`` under the key ``(seed's low
word, seed's high word)`` - anyone can recompute a draw from the logits.
"""
from dataclasses import dataclass
from typing import Optional

import torch

from ..ops import kernels as K


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 1.0
    top_k: Optional[int] = None
    seed: int = 1234

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if self.top_k is not None and self.top_k < 1:
            raise ValueError("top_k must be at least 1")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0


def sample(logits: torch.Tensor, params: SamplingParams, row_keys: torch.Tensor,
           positions: Optional[torch.Tensor], position_offset: int = 0,
           out: Optional[torch.Tensor] = None, probs: Optional[torch.Tensor] = None,
           seed_words: Optional[torch.Tensor] = None):
    """int32 [B] next tokens for float32 logits [B, V].  ``row_keys`` (int32 [B])
    identifies each row's request and ``positions`` (+ offset) the place of the token
    being drawn; both only feed the noise.  ``seed_words`` (int32 [2] on the device: the
    seed's low and high word) replaces ``params.seed`` where the launch is recorded and
    replayed for other seeds."""
    if params.greedy and probs is None:
        return K.argmax(logits, out=out)
    if params.greedy:
        # probabilities of the reference's near-one-hot law, token by exact argmax
        K.sample(logits, 1e-5, params.top_k, params.seed, row_keys, positions,
                 position_offset, out=None, probs=probs)
        return K.argmax(logits, out=out)
    return K.sample(logits, params.temperature, params.top_k, params.seed, row_keys,
                    positions, position_offset, out=out, probs=probs, seed_words=seed_words)


def seed_words(seed: int):
    """The low and high 32-bit word of a seed as the signed integers an int32 buffer holds."""
    def signed(u):
        return u - (1 << 32) if u >= (1 << 31) else u
    seed &= (1 << 64) - 1
    return signed(seed & 0xFFFFFFFF), signed(seed >> 32)


def logits_to_probs(logits: torch.Tensor, temperature: float = 1.0,
                    top_k: Optional[int] = None) -> torch.Tensor:
    """float32 [B, V] probabilities the sampler draws from (generate.py:44-52)."""
    B, V = logits.shape
    probs = torch.empty((B, V), dtype=torch.float32, device=logits.device)
    keys = torch.zeros(B, dtype=torch.int32, device=logits.device)
    K.sample(logits, temperature, top_k, 0, keys, None, 0, probs=probs)
    return probs
