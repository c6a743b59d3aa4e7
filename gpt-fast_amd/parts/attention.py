"""Causal attention with grouped key/value heads over the paged cache
(reference model.py:167-216)."""
import torch

from ..cache.store import KVNeed
from ..config.spec import AttentionSpec
from ..ops import attention as A
from ..ops import kernels as K
from ..ops import linear as L
from .base import POSITIONS, Param, Part, Runtime, add_late, check_bound, register_mixer


class Attention(Part):
    """``wo( softmax(q k^T * scale + causal mask) v )`` with q, k, v = split(wqkv x),
    positions applied to q and k by the spec's position encoding, k and v written to the
    cache entry before they are read.  Query head h reads kv head h // (H / Hkv)
    (model.py:209-210).  Scores, softmax and the weighted sum are float32."""

    def __init__(self, spec: AttentionSpec, runtime: Runtime):
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError(f"{spec.n_heads} heads do not divide into {spec.n_kv_heads} kv heads")
        self.spec = spec
        self.rt = runtime
        self.position = POSITIONS.build(spec.position, runtime)
        self.scale = spec.scale if spec.scale is not None else K.default_scale(spec.head_dim)
        self.window = 0 if spec.window is None else int(spec.window)
        self.wqkv = self.wo = None

    def parameters(self):
        s = self.spec
        return {"wqkv": Param(((s.n_heads + 2 * s.n_kv_heads) * s.head_dim, s.dim)),
                "wo": Param((s.dim, s.n_heads * s.head_dim))}

    def bind(self, tensors):
        check_bound("Attention", self.parameters(), tensors)
        self.wqkv, self.wo = tensors["wqkv"], tensors["wo"]

    def cache_need(self):
        s = self.spec
        return KVNeed(s.n_kv_heads, s.head_dim, s.window)

    @property
    def replayable(self):
        return bool(getattr(self.position, "replayable", False))

    def step_flops(self, q_lens, starts) -> float:
        """Multiply-adds times two of a step that brings ``q_lens[b]`` tokens to sequences
        that hold ``starts[b]``: the two projections, and scores and weighted sums over the
        keys each token sees (a causal prompt counts its triangle, not the square)."""
        s = self.spec
        n = sum(q_lens)
        flops = 2.0 * n * (self.wqkv_rows() + s.n_heads * s.head_dim) * s.dim
        for q, start in zip(q_lens, starts):
            keys = q * start + q * (q + 1) / 2.0
            if s.window is not None:
                keys = min(keys, q * float(s.window))
            flops += 2.0 * 2.0 * s.n_heads * s.head_dim * keys
        return flops

    def wqkv_rows(self) -> int:
        s = self.spec
        return (s.n_heads + 2 * s.n_kv_heads) * s.head_dim

    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream
    takes_prepared = True          # x may be an ops.linear.HalfNormed

    def forward(self, x, batch, entry, residual):
        s = self.spec
        n_rows = x.shape[0]
        q = None
        fused = getattr(self.position, "project_rotate_store", None)
        if fused is not None and L.can_project_rotate_store(x, self.wqkv, s.head_dim):
            # few rows: projection, rotation and cache write in one kernel
            q = fused(x, self.wqkv, batch, entry, s.n_heads, s.n_kv_heads, s.head_dim)
        if q is None:
            qkv = L.linear(x, self.wqkv,                                    # model.py:195
                           may_stay_sliced=getattr(self.position, "takes_sliced", False))
            whole = getattr(self.position, "rotate_store_attend", None)
            if whole is not None and isinstance(qkv, L.SlicedRows):
                # one token per sequence, the projection still in slices: rotation, cache
                # write and attention as one kernel (model.py:201-211)
                y = whole(qkv, batch, entry, s.n_heads, s.n_kv_heads, s.head_dim, self.scale,
                          self.window)
                if y is not None:
                    y = y.view(n_rows, s.n_heads * s.head_dim)
                    add_late(residual, lambda rows, then_norm, takes_halves: L.linear_into(
                        y, self.wo, rows, then_norm, takes_halves))           # model.py:215, 162
                    return
            q = self.position.rotate_and_store(qkv, batch, entry, s.n_heads, s.n_kv_heads,
                                               s.head_dim)                  # model.py:201-207

        def finish(rows, then_norm, takes_halves):
            # the output projection may take the heads' results in the order it loads them in
            rows_for_wo = L.takes_chunked_rows(n_rows, q.dtype, self.wo, then_norm, takes_halves)
            y = A.attention(q, entry.k_pages, entry.v_pages, batch, batch.table(entry.group_id),
                            self.scale, self.window, for_product=rows_for_wo)   # model.py:209-211
            if isinstance(y, torch.Tensor):
                y = y.view(n_rows, s.n_heads * s.head_dim)
            return L.linear_into(y, self.wo, rows, then_norm, takes_halves)  # model.py:215, 162

        add_late(residual, finish)


register_mixer("attention", Attention)
