"""Python faces of the HIP kernels: shape checks on the host, then the launch.

Every function takes device tensors, launches on torch's current stream and returns
its output tensor.  Shapes are checked here because the kernels trust them.  "bf16" in
an argument list is decided by the tensors' dtype; float32 and bfloat16 are the only
activation types.
"""
import ctypes
import math
from typing import Optional

import torch

from .library import (KernelError, check, library, ptr, require_contiguous, require_device,
                      stream_handle)

PAGE = 64          # tokens per cache page; equals GFA_PAGE of csrc/common.h

_i = ctypes.c_int
_f = ctypes.c_float
_sz = ctypes.c_size_t


def _is_bf16(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise KernelError(f"activation dtype {t.dtype}: float32 or bfloat16 only")


def _want(t, dtype, name):
    if t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, is {t.dtype}")


# ----------------------------------------------------------------------------- embedding
def embed(table: torch.Tensor, tokens: torch.Tensor, out: Optional[torch.Tensor] = None):
    """out[n, :] = float(table[tokens[n], :]); table [V, D], tokens int32 [N]."""
    require_device(table, tokens)
    require_contiguous(table=table, tokens=tokens)
    _want(tokens, torch.int32, "tokens")
    n, dim = tokens.numel(), table.shape[1]
    if out is None:
        out = torch.empty((n, dim), dtype=torch.float32, device=table.device)
    elif out.shape != (n, dim) or out.dtype != torch.float32 or not out.is_contiguous():
        raise KernelError("embed: out must be contiguous float32 [n_tokens, dim]")
    check(library("core").gfa_embed(ptr(table), _i(_is_bf16(table)), ptr(tokens), ptr(out),
                                    _i(n), _i(dim), stream_handle()), "embed")
    return out


# ----------------------------------------------------------------------------- norm
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None):
    """out[i] = x[r] * rsqrt(mean(x[r]^2) + eps) * weight, r = rows[i] if rows else i.
    x float32 [N, D]; weight float32 [D]."""
    require_device(x, weight, rows)
    require_contiguous(x=x, weight=weight, rows=rows)
    _want(x, torch.float32, "x")
    _want(weight, torch.float32, "norm weight")
    dim = x.shape[-1]
    if weight.numel() != dim:
        raise KernelError(f"rmsnorm: weight has {weight.numel()} elements, rows have {dim}")
    n = x.numel() // dim if rows is None else rows.numel()
    if rows is not None:
        _want(rows, torch.int32, "rows")
    if out is None:
        out = torch.empty((n, dim), dtype=out_dtype, device=x.device)
    elif out.shape != (n, dim) or out.dtype != out_dtype or not out.is_contiguous():
        raise KernelError("rmsnorm: out has the wrong shape or dtype")
    check(library("core").gfa_rmsnorm(ptr(x), ptr(weight), ptr(rows), ptr(out),
                                      _i(_is_bf16(out)), _i(n), _i(dim), _f(eps),
                                      stream_handle()), "rmsnorm")
    return out


# ----------------------------------------------------------------------------- float32 product
def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
             accumulate: bool = False):
    """out[m, n] (+)= sum_k a[m, k] w[n, k], all float32; a [M, K], w [N, K]."""
    require_device(a, w, out)
    _want(a, torch.float32, "a")
    _want(w, torch.float32, "w")
    require_contiguous(w=w)
    if a.dim() != 2 or w.dim() != 2 or a.shape[1] != w.shape[1]:
        raise KernelError(f"gemm_f32: a {tuple(a.shape)} and w {tuple(w.shape)} do not fit")
    if a.stride(1) != 1:
        raise KernelError("gemm_f32: a must have unit stride along k")
    M, K = a.shape
    N = w.shape[0]
    if out is None:
        if accumulate:
            raise KernelError("gemm_f32: accumulate needs an out tensor")
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    elif out.shape != (M, N) or out.dtype != torch.float32 or out.stride(1) != 1:
        raise KernelError("gemm_f32: out must be float32 [M, N] with unit column stride")
    check(library("core").gfa_gemm_f32(ptr(a), ptr(w), ptr(out), _i(M), _i(N), _i(K),
                                       _i(a.stride(0)), _i(out.stride(0)),
                                       _i(1 if accumulate else 0), stream_handle()), "gemm_f32")
    return out


def gemm_bf16_naive(a: torch.Tensor, w: torch.Tensor):
    """Plain counterpart of the bfloat16 products: float32 out[m, n] = sum_k a[m,k] w[n,k]."""
    require_device(a, w)
    require_contiguous(a=a, w=w)
    _want(a, torch.bfloat16, "a")
    _want(w, torch.bfloat16, "w")
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise KernelError("gemm_bf16_naive: inner sizes differ")
    out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    check(library("core").gfa_gemm_bf16_naive(ptr(a), ptr(w), ptr(out), _i(M), _i(N), _i(K),
                                              stream_handle()), "gemm_bf16_naive")
    return out


# ----------------------------------------------------------------------------- rope + cache
def _check_pages(k_pages, v_pages, n_kv_heads, head_dim, dtype):
    for name, p, tail in (("k_pages", k_pages, (n_kv_heads, PAGE, head_dim)),
                          ("v_pages", v_pages, (n_kv_heads, head_dim, PAGE))):
        if p is None:
            continue
        if p.dim() != 4 or tuple(p.shape[1:]) != tail:
            raise KernelError(f"{name} must be [n_pages, {tail[0]}, {tail[1]}, {tail[2]}], "
                              f"is {tuple(p.shape)}")
        if p.dtype != dtype or not p.is_contiguous():
            raise KernelError(f"{name} must be contiguous {dtype}")


def rope_cache_write(qkv: torch.Tensor, freqs: Optional[torch.Tensor], tok_seq, tok_pos, table,
                     k_pages, v_pages, n_heads: int, n_kv_heads: int, head_dim: int,
                     rotary_dim: int, layout: int, q_out: Optional[torch.Tensor] = None):
    """Rotate q and k of qkv [N, (H+2G)*hd] by position, write q to q_out [N, H, hd] and
    k, v into the pages (skipped if k_pages is None).  rotary_dim 0: no rotation."""
    require_device(qkv, freqs, tok_seq, tok_pos, table, k_pages, v_pages)
    require_contiguous(qkv=qkv, freqs=freqs, tok_seq=tok_seq, tok_pos=tok_pos, table=table)
    n = qkv.shape[0]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    if qkv.dim() != 2 or qkv.shape[1] != width:
        raise KernelError(f"rope: qkv is {tuple(qkv.shape)}, expected [N, {width}]")
    if head_dim % 2 or rotary_dim % 2 or not 0 <= rotary_dim <= head_dim:
        raise KernelError(f"rope: head_dim {head_dim} and rotary_dim {rotary_dim} must be "
                          f"even, rotary_dim <= head_dim")
    if rotary_dim:
        _want(freqs, torch.float32, "freqs")
        if freqs.numel() != rotary_dim // 2:
            raise KernelError(f"rope: {freqs.numel()} frequencies for rotary_dim {rotary_dim}")
    if tok_seq.numel() < n or tok_pos.numel() < n:
        raise KernelError("rope: token maps are shorter than the batch")
    _want(tok_seq, torch.int32, "tok_seq")
    _want(tok_pos, torch.int32, "tok_pos")
    _want(table, torch.int32, "table")
    if (k_pages is None) != (v_pages is None):
        raise KernelError("rope: give both k_pages and v_pages, or neither")
    _check_pages(k_pages, v_pages, n_kv_heads, head_dim, qkv.dtype)
    if q_out is None:
        q_out = torch.empty((n, n_heads, head_dim), dtype=qkv.dtype, device=qkv.device)
    elif q_out.numel() != n * n_heads * head_dim or q_out.dtype != qkv.dtype:
        raise KernelError("rope: q_out has the wrong size or dtype")
    check(library("core").gfa_rope_cache_write(
        ptr(qkv), ptr(q_out), ptr(k_pages), ptr(v_pages), ptr(freqs), ptr(tok_seq), ptr(tok_pos),
        ptr(table), _i(table.shape[1]), _i(n), _i(n_heads), _i(n_kv_heads), _i(head_dim),
        _i(rotary_dim), _i(layout), _i(_is_bf16(qkv)), stream_handle()), "rope_cache_write")
    return q_out


def rope_cache_write_sliced(part: torch.Tensor, freqs: Optional[torch.Tensor], tok_seq, tok_pos, table,
                            k_pages, v_pages, n_heads: int, n_kv_heads: int, head_dim: int,
                            rotary_dim: int):
    """:func:`rope_cache_write` for rows given as the float partial sums of a sliced product,
    part [S, N, (H+2G)*hd]: slices added in order, pairs (2i, 2i+1) rotated, bfloat16 q
    returned and k, v stored.  head_dim and rotary_dim multiples of 8."""
    require_device(part, freqs, tok_seq, tok_pos, table, k_pages, v_pages)
    require_contiguous(part=part, freqs=freqs, tok_seq=tok_seq, tok_pos=tok_pos, table=table)
    _want(part, torch.float32, "part")
    width = (n_heads + 2 * n_kv_heads) * head_dim
    if part.dim() != 3 or part.shape[2] != width:
        raise KernelError(f"rope: the partial sums are {tuple(part.shape)}, expected [S, N, {width}]")
    S, n, _ = part.shape
    if head_dim % 8 or rotary_dim % 8 or not 0 <= rotary_dim <= head_dim:
        raise KernelError("rope over partial sums: head_dim and rotary_dim in multiples of 8")
    if rotary_dim:
        _want(freqs, torch.float32, "freqs")
        if freqs.numel() != rotary_dim // 2:
            raise KernelError(f"rope: {freqs.numel()} frequencies for rotary_dim {rotary_dim}")
    if tok_seq.numel() < n or tok_pos.numel() < n:
        raise KernelError("rope: token maps are shorter than the batch")
    for name, t in (("tok_seq", tok_seq), ("tok_pos", tok_pos), ("table", table)):
        _want(t, torch.int32, name)
    if (k_pages is None) != (v_pages is None):
        raise KernelError("rope: give both k_pages and v_pages, or neither")
    _check_pages(k_pages, v_pages, n_kv_heads, head_dim, torch.bfloat16)
    q_out = torch.empty((n, n_heads, head_dim), dtype=torch.bfloat16, device=part.device)
    check(library("core").gfa_rope_cache_write_sliced(
        ptr(part), _i(S), ptr(q_out), ptr(k_pages), ptr(v_pages), ptr(freqs), ptr(tok_seq),
        ptr(tok_pos), ptr(table), _i(table.shape[1]), _i(n), _i(n_heads), _i(n_kv_heads),
        _i(head_dim), _i(rotary_dim), stream_handle()), "rope_cache_write_sliced")
    return q_out


# ----------------------------------------------------------------------------- attention
def attention_generic(q: torch.Tensor, k_pages, v_pages, tok_seq, tok_pos, table,
                      scale: float, window: int = 0, out: Optional[torch.Tensor] = None):
    """Each token's heads attend to keys lo..pos of its sequence's pages; q [N, H, hd]."""
    require_device(q, k_pages, v_pages, tok_seq, tok_pos, table)
    require_contiguous(q=q, tok_seq=tok_seq, tok_pos=tok_pos, table=table)
    n, H, hd = q.shape
    G = k_pages.shape[1]
    if H % G:
        raise KernelError(f"attention: {H} heads do not divide into {G} kv heads")
    if hd > 512:
        raise KernelError(f"attention: head_dim {hd} > 512 is not supported")
    _check_pages(k_pages, v_pages, G, hd, q.dtype)
    _want(tok_seq, torch.int32, "tok_seq")
    _want(tok_pos, torch.int32, "tok_pos")
    _want(table, torch.int32, "table")
    if tok_seq.numel() < n or tok_pos.numel() < n:
        raise KernelError("attention: token maps are shorter than the batch")
    if out is None:
        out = torch.empty_like(q)
    check(library("core").gfa_attention_generic(
        ptr(q), ptr(k_pages), ptr(v_pages), ptr(tok_seq), ptr(tok_pos), ptr(table),
        _i(table.shape[1]), ptr(out), _i(n), _i(H), _i(G), _i(hd), _f(scale), _i(window),
        _i(_is_bf16(q)), stream_handle()), "attention_generic")
    return out


# ----------------------------------------------------------------------------- elementwise
def silu_mul(gu: torch.Tensor, out: Optional[torch.Tensor] = None):
    """out[n, i] = silu(gu[n, i]) * gu[n, I + i]; gu [N, 2I]."""
    require_device(gu)
    require_contiguous(gu=gu)
    n, two_i = gu.shape
    if two_i % 2:
        raise KernelError("silu_mul: the row width must be even")
    if out is None:
        out = torch.empty((n, two_i // 2), dtype=gu.dtype, device=gu.device)
    check(library("core").gfa_silu_mul(ptr(gu), ptr(out), _i(n), _i(two_i // 2),
                                       _i(_is_bf16(gu)), stream_handle()), "silu_mul")
    return out


def add_into(residual: torch.Tensor, y: torch.Tensor):
    """residual += float(y), residual float32."""
    require_device(residual, y)
    require_contiguous(residual=residual, y=y)
    _want(residual, torch.float32, "residual")
    if residual.numel() != y.numel():
        raise KernelError("add_into: sizes differ")
    check(library("core").gfa_add_into(ptr(residual), ptr(y), _sz(y.numel()), _i(_is_bf16(y)),
                                       stream_handle()), "add_into")
    return residual


def scale_cap(x: torch.Tensor, scale: float = 1.0, cap: float = 0.0):
    """In place on float32 ``x``: x * scale, then cap * tanh(x / cap) if cap > 0."""
    require_device(x)
    require_contiguous(x=x)
    _want(x, torch.float32, "x")
    check(library("core").gfa_scale_cap(ptr(x), _sz(x.numel()), _f(scale), _f(cap),
                                        stream_handle()), "scale_cap")
    return x


def add_rmsnorm(residual: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float):
    """residual += float(y), then the RMS norm of the new rows in bfloat16: one pass.
    residual float32 [N, D], y bfloat16 [N, D], weight float32 [D]."""
    require_device(residual, y, weight)
    require_contiguous(residual=residual, y=y, weight=weight)
    _want(residual, torch.float32, "residual")
    _want(weight, torch.float32, "norm weight")
    _want(y, torch.bfloat16, "y")
    if residual.dim() != 2 or y.shape != residual.shape or weight.numel() != residual.shape[1]:
        raise KernelError("add_rmsnorm: shapes of residual, y and the norm weight do not fit")
    out = torch.empty(residual.shape, dtype=torch.bfloat16, device=residual.device)
    check(library("core").gfa_add_rmsnorm(ptr(residual), ptr(y), ptr(weight), ptr(out),
                                          _i(residual.shape[0]), _i(residual.shape[1]), _f(eps),
                                          stream_handle()), "add_rmsnorm")
    return out


# ----------------------------------------------------------------------------- sampling
# vocabularies beyond this are spread over many workgroups per row
SPLIT_SAMPLING_ABOVE = 16384


_split_workspaces = {}


def _device_index(device) -> int:
    dev = torch.device(device)
    return torch.cuda.current_device() if dev.index is None else dev.index


def _split_workspace(B: int, V: int, device) -> torch.Tensor:
    """The workspace of the many-workgroup sampler for this many rows: allocated and zeroed
    once per device, stream and size.  The kernels of a call leave its histograms zero again, so it is
    used call after call and recorded launches keep a valid address; calls on different
    streams get workspaces of their own, and a call whose launch failed drops its workspace
    (its histograms may be left half counted)."""
    key = (_device_index(device), torch.cuda.current_stream().cuda_stream
           if not torch.cuda.is_current_stream_capturing() else "capture", B, V)
    ws = _split_workspaces.get(key)
    if ws is None and key[1] == "capture":
        # a recording replays on whatever stream; it uses the workspace its warm-up run made
        for (dev, _, b, v), t in _split_workspaces.items():
            if (dev, b, v) == (key[0], B, V):
                return t
        raise KernelError("the sampler's workspace must exist before a step is recorded: "
                          "run the step once outside the recording")
    if ws is None:
        lib = library("sampling")
        lib.gfa_sample_split_workspace.restype = ctypes.c_size_t
        n = lib.gfa_sample_split_workspace(_i(B), _i(V))
        ws = torch.zeros(n // 4, dtype=torch.int32, device=torch.device("cuda", key[0]))
        _split_workspaces[key] = ws
    return ws


def _sample_split(logits, temperature, top_k, seed, seed_words, row_keys, positions,
                  position_offset, out, probs):
    B, V = logits.shape
    ws = _split_workspace(B, V, logits.device)
    code = library("sampling").gfa_sample_split(
        ptr(logits), _sz(logits.stride(0)), _i(B), _i(V), _f(temperature), _i(top_k),
        ctypes.c_uint64(seed & (2 ** 64 - 1)), ptr(seed_words), ptr(row_keys), ptr(positions),
        _i(position_offset), ptr(out), ptr(probs), ptr(ws), stream_handle())
    if code != 0:
        for key in [k for k, t in _split_workspaces.items() if t is ws]:
            del _split_workspaces[key]
    check(code, "sample_split")
    return out


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None):
    """int32 [B]: index of the largest of each row of float32 logits [B, V]."""
    require_device(logits)
    _want(logits, torch.float32, "logits")
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax: logits must be [B, V] with unit column stride")
    B, V = logits.shape
    if out is None:
        out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    if V > SPLIT_SAMPLING_ABOVE:
        return _sample_split(logits, 0.0, 0, 0, None, None, None, 0, out, None)
    check(library("sampling").gfa_argmax(ptr(logits), ptr(out), _i(B), _i(V),
                                         _sz(logits.stride(0)), stream_handle()), "argmax")
    return out


def sample(logits: torch.Tensor, temperature: float, top_k: Optional[int], seed: int,
           row_keys: torch.Tensor, positions: Optional[torch.Tensor], position_offset: int = 0,
           out: Optional[torch.Tensor] = None, probs: Optional[torch.Tensor] = None,
           seed_words: Optional[torch.Tensor] = None):
    """int32 [B]: one draw per row from softmax(top_k(logits / max(temperature, 1e-5))).
    ``seed_words``: int32 [2] on the device, the seed's low and high word; if given it
    replaces ``seed`` (a recorded launch then follows the buffer's contents)."""
    require_device(logits, row_keys, positions, probs, seed_words)
    if seed_words is not None and (seed_words.dtype != torch.int32 or seed_words.numel() < 2
                                   or not seed_words.is_contiguous()):
        raise KernelError("sample: seed_words must be contiguous int32 [2]")
    _want(logits, torch.float32, "logits")
    _want(row_keys, torch.int32, "row_keys")
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample: logits must be [B, V] with unit column stride")
    B, V = logits.shape
    if row_keys.numel() < B or (positions is not None and positions.numel() < B):
        raise KernelError("sample: row_keys / positions are shorter than the batch")
    if positions is not None:
        _want(positions, torch.int32, "positions")
    if probs is not None and (probs.shape != (B, V) or probs.dtype != torch.float32
                              or not probs.is_contiguous()):
        raise KernelError("sample: probs must be contiguous float32 [B, V]")
    if out is None:
        out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    k = 0 if top_k is None else int(top_k)
    if k < 0:
        raise KernelError("sample: top_k must be positive")
    if V > SPLIT_SAMPLING_ABOVE:
        if temperature <= 0:
            raise KernelError("sample: temperature must be positive (greedy is argmax)")
        return _sample_split(logits, temperature, k, seed, seed_words, row_keys, positions,
                             position_offset, out, probs)
    check(library("sampling").gfa_sample(
        ptr(logits), _sz(logits.stride(0)), _i(B), _i(V), _f(temperature), _i(k),
        ctypes.c_uint64(seed & (2 ** 64 - 1)), ptr(seed_words), ptr(row_keys), ptr(positions),
        _i(position_offset), ptr(out), ptr(probs), stream_handle()), "sample")
    return out


def default_scale(head_dim: int) -> float:
    return 1.0 / math.sqrt(head_dim)
