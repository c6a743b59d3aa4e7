"""Position encodings of attention.

A position encoding turns the fused projection ``qkv`` of a step into rotated queries and
writes keys and values into the cache entry.  Rotary encodings differ only in their
frequency vector, pair layout and rotary width, all parameters of one kernel.
"""
import math

import torch

from ..config.spec import PositionSpec
from ..ops import kernels as K
from ..ops import linear as L
from .base import Part, Runtime, register_position


def rotary_frequencies(rotary_dim: int, base: float) -> torch.Tensor:
    """f_i = 1 / base^(2i / rotary_dim) in float32 (reference model.py:271)."""
    idx = torch.arange(0, rotary_dim, 2)[: rotary_dim // 2].float()
    return 1.0 / (base ** (idx / rotary_dim))


def llama3_scaled(freqs: torch.Tensor, factor: float, low_freq_factor: float,
                  high_freq_factor: float, original_max_position_embeddings: float,
                  **_ignored) -> torch.Tensor:
    """Llama-3.1 rescale by wavelength (reference model.py:244-263): wavelengths below
    orig/high are kept, above orig/low divided by ``factor``, between blended."""
    orig = original_max_position_embeddings
    low_wavelen = orig / low_freq_factor
    high_wavelen = orig / high_freq_factor
    wavelen = 2 * math.pi / freqs
    if high_freq_factor == low_freq_factor:
        blended = freqs
    else:
        smooth = (orig / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
        blended = (1 - smooth) * freqs / factor + smooth * freqs
    return torch.where(wavelen < high_wavelen, freqs,
                       torch.where(wavelen > low_wavelen, freqs / factor, blended))


FREQUENCY_SCALINGS = {"llama3": llama3_scaled}


class RotaryPosition(Part):
    LAYOUTS = {"interleaved": 0, "half": 1}
    replayable = True

    def __init__(self, spec: PositionSpec, runtime: Runtime):
        if spec.layout not in self.LAYOUTS:
            raise ValueError(f"rotary layout '{spec.layout}': {sorted(self.LAYOUTS)}")
        if spec.rotary_dim <= 0 or spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be positive and even")
        self.spec = spec
        self.rt = runtime
        freqs = rotary_frequencies(spec.rotary_dim, spec.base)
        scaling = spec.scaling_dict()
        if scaling is not None:
            kind = scaling.get("rope_type")
            if kind not in FREQUENCY_SCALINGS:
                raise ValueError(f"rope scaling '{kind}': {sorted(FREQUENCY_SCALINGS)}")
            freqs = FREQUENCY_SCALINGS[kind](
                freqs, **{k: v for k, v in scaling.items() if k != "rope_type"})
        self.freqs_host = freqs.to(torch.float32)
        self.freqs = self.freqs_host.to(runtime.device)

    # qkv may come as ops.linear.SlicedRows (a sliced product's partial sums): they are added
    # on the way where the kernel for that fits
    takes_sliced = True

    def rotate_and_store(self, qkv, batch, entry, n_heads, n_kv_heads, head_dim):
        write = entry is not None and entry.writes
        pages = (entry.k_pages if write else None, entry.v_pages if write else None)
        if isinstance(qkv, L.SlicedRows):
            if (self.spec.layout == "interleaved" and qkv.dtype == torch.bfloat16
                    and head_dim % 8 == 0 and self.spec.rotary_dim % 8 == 0):
                return K.rope_cache_write_sliced(
                    qkv.part, self.freqs, batch.tok_seq, batch.tok_pos, batch.table(entry.group_id),
                    *pages, n_heads, n_kv_heads, head_dim, self.spec.rotary_dim)
            qkv = qkv.rows()
        return K.rope_cache_write(
            qkv, self.freqs, batch.tok_seq, batch.tok_pos, batch.table(entry.group_id), *pages,
            n_heads, n_kv_heads, head_dim, self.spec.rotary_dim, self.LAYOUTS[self.spec.layout])

    def rotate_store_attend(self, qkv, batch, entry, n_heads, n_kv_heads, head_dim, scale, window):
        """For a step of one token per sequence whose ``qkv`` is still an
        ``ops.linear.SlicedRows``: rotation, cache write and attention in one kernel.  None:
        not available for this step (the caller rotates, stores and attends apart)."""
        # a run that reads another run's cache attends to that run's keys and values, also at
        # the token's own position: not to the ones this kernel would make of its own rows
        if (self.spec.layout != "interleaved" or not isinstance(qkv, L.SlicedRows)
                or qkv.dtype != torch.bfloat16 or entry is None or not entry.writes):
            return None
        from ..ops import attention_bf16 as AB
        return AB.attention_sliced(qkv.part, self.freqs, self.spec.rotary_dim, entry.k_pages,
                                   entry.v_pages, True, batch, batch.table(entry.group_id),
                                   scale, window or 0, n_heads)

    def project_rotate_store(self, x, wqkv, batch, entry, n_heads, n_kv_heads, head_dim):
        """Projection + rotation + cache write in one kernel for few rows (interleaved
        pairs only: both elements of a pair are then in one lane).  None: not available."""
        if self.spec.layout != "interleaved":
            return None
        write = entry is not None and entry.writes
        return L.qkv_rope_store(
            x, wqkv, self.freqs, batch.tok_seq, batch.tok_pos,
            batch.table(entry.group_id), entry.k_pages if write else None,
            entry.v_pages if write else None, n_heads, n_kv_heads, head_dim, self.spec.rotary_dim)


class NoPosition(Part):
    """No position information: q, k, v pass through unchanged into q and the cache."""
    replayable = True

    def __init__(self, spec: PositionSpec, runtime: Runtime):
        self.spec = spec

    def rotate_and_store(self, qkv, batch, entry, n_heads, n_kv_heads, head_dim):
        write = entry is not None and entry.writes
        return K.rope_cache_write(
            qkv, None, batch.tok_seq, batch.tok_pos, batch.table(entry.group_id),
            entry.k_pages if write else None, entry.v_pages if write else None,
            n_heads, n_kv_heads, head_dim, 0, 0)


register_position("rope", RotaryPosition)
register_position("none", NoPosition)
