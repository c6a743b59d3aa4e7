"""Python face of the matrix-core attention kernel (csrc/attention_bf16.hip)."""
import ctypes

import torch

from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i = ctypes.c_int
_f = ctypes.c_float

MAX_SPLITS = 32
# Single-token steps.  A wave takes its keys one 32-key block after another (0.6 us each, two
# in flight); splitting a context over several workgroups shortens that chain but costs a
# second kernel that sums the splits (3 to 4 us with its boundary).  Measured on contexts of
# 128 to 16,384 keys and 1 to 64 sequences (8 kv heads, head size 128, 256 compute units): no
# split pays while a wave has at most SPLIT_FROM_BLOCKS blocks; a workgroup on every second
# compute unit already streams the cache at the memory's rate, so splits only make up for
# missing workgroups, never beyond one per compute unit; a split is left with two blocks per
# wave at least.
SPLIT_FROM_BLOCKS = 6
LONG_BLOCKS = 48           # with a workgroup on every second compute unit or more, two splits
                           # from this many blocks per wave on

_units = {}


def compute_units(device=None) -> int:
    """Compute units of the device (asked once each)."""
    index = torch.cuda.current_device() if device is None else torch.device(device).index
    n = _units.get(index)
    if n is None:
        n = _units[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return n


TILED_MIN_ROWS = 64        # prompts with at least this many (token, head) rows per kv head use
                           # the workgroup-tiled kernel (keys and values through LDS)
PREFILL_ROW_TILES = 4      # 16-row tiles per wave for prompts
TILED_ROW_TILES = 0        # of the workgroup-tiled kernel: 1 or 2, or 0 = by the size of the grid


def plan(n_seqs: int, max_q_len: int, H: int, G: int, hd: int, table_width: int, units=None):
    """(row tiles per wave, waves per workgroup, workgroups per sequence and kv head,
    context splits) for a step on a device of ``units`` compute units (default: the current
    device's)."""
    R = H // G
    if max_q_len == 1:
        fill = units or compute_units()
        streaming = (fill + 1) // 2
        rt = 1
        nw = 4 if hd <= 128 else 2
        tiles = (R + 15) // 16
        groups = n_seqs * G * tiles                      # workgroups without any split
        blocks = (table_width * 2 + nw - 1) // nw          # key blocks per wave at most
        if blocks <= SPLIT_FROM_BLOCKS or groups >= fill:
            splits = 1
        elif groups >= streaming:
            splits = 2 if blocks >= LONG_BLOCKS else 1
        else:
            splits = min((blocks + 1) // 2, (fill + groups - 1) // groups, MAX_SPLITS)
        return rt, nw, tiles, splits
    rt = PREFILL_ROW_TILES if hd <= 128 else min(PREFILL_ROW_TILES, 2)
    rows = max_q_len * R
    if rows <= 16:
        rt = 1
    elif rows <= 32:
        rt = min(rt, 2)
    return rt, 1, (rows + 16 * rt - 1) // (16 * rt), 1


def attention(q, k_pages, v_pages, batch, table, scale, window, chunked: bool = False):
    """The kernel's result [N, H, hd], or None if it does not take this shape (head sizes
    that are no multiple of 16 or exceed 256 go to the plain kernel).  ``chunked``: where the
    step is one token for each of up to 64 sequences, the result [N, H * hd] is returned as
    ``gemm_bf16.ChunkedRows``, the order in which the few-row product that follows loads it."""
    n, H, hd = q.shape
    G = k_pages.shape[1]
    if hd % 16 or hd > 256 or H % G:
        return None
    require_device(q, k_pages, v_pages, table, batch.q_start, batch.start_pos)
    require_contiguous(q=q, k_pages=k_pages, v_pages=v_pages, table=table)
    if q.dtype != torch.bfloat16 or k_pages.dtype != torch.bfloat16 or v_pages.dtype != torch.bfloat16:
        raise KernelError("attention_bf16: bfloat16 tensors only")
    if tuple(k_pages.shape[1:]) != (G, 64, hd) or tuple(v_pages.shape[1:]) != (G, hd, 64):
        raise KernelError(f"attention_bf16: pages are {tuple(k_pages.shape)} / {tuple(v_pages.shape)}")
    if batch.q_start.numel() != batch.n_seqs + 1 or batch.start_pos.numel() != batch.n_seqs \
            or table.shape[0] != batch.n_seqs or table.dtype != torch.int32:
        raise KernelError("attention_bf16: the batch description does not fit its sequences")
    R = H // G
    if batch.max_q_len * R >= TILED_MIN_ROWS and hd <= 128:
        out = torch.empty_like(q)
        check(library("attention_bf16").gfa_attention_tiled_bf16(
            ptr(q), ptr(k_pages), ptr(v_pages), ptr(batch.q_start), ptr(batch.start_pos),
            ptr(table), _i(table.shape[1]), ptr(out), _i(n), _i(batch.n_seqs), _i(H), _i(G), _i(hd),
            _f(scale), _i(window), _i(batch.max_q_len * R), _i(TILED_ROW_TILES), stream_handle()),
            "attention_tiled_bf16")
        return out
    rt, nw, tiles, splits = plan(batch.n_seqs, batch.max_q_len, H, G, hd, table.shape[1])
    one_each = batch.max_q_len == 1 and n == batch.n_seqs
    chunked = chunked and one_each and n <= 64 and tiles == 1
    if chunked:
        from .gemm_bf16 import ChunkedRows
        res = ChunkedRows(n, H * hd, q.device)
        out = res.data
    else:
        res = out = torch.empty_like(q)
    ws_o = ws_ml = None
    if splits > 1:
        ws_o = torch.empty((splits, n * H, hd), dtype=torch.float32, device=q.device)
        ws_ml = torch.empty((splits, n * H, 2), dtype=torch.float32, device=q.device)
    check(library("attention_bf16").gfa_attention_bf16(
        ptr(q), ptr(k_pages), ptr(v_pages), ptr(batch.q_start), ptr(batch.start_pos), ptr(table),
        _i(table.shape[1]), ptr(out), ptr(ws_o), ptr(ws_ml), _i(n), _i(batch.n_seqs), _i(H), _i(G),
        _i(hd), _f(scale), _i(window), _i(rt), _i(nw), _i(tiles), _i(splits),
        _i(int(one_each)), _i(int(chunked)), stream_handle()),
        "attention_bf16")
    return res


def attention_sliced(part, freqs, rot: int, k_pages, v_pages, write_cache: bool, batch, table,
                     scale: float, window: int, H: int):
    """One token per sequence whose q, k and v rows are still the float32 partial sums ``part``
    [S, N, (H + 2 G) * hd] of a sliced product: the slices are added, queries and keys rotated
    (interleaved pairs; ``freqs`` [rot / 2]), the new keys and values written to the cache
    (unless ``write_cache`` is false) and attended, in one kernel.  Returns [N, H, hd]
    bfloat16, or None if the kernel does not take this step (the caller then rotates and
    attends with the kernels of their own)."""
    S, n, width = part.shape
    G = k_pages.shape[1]
    hd = width // (H + 2 * G) if H + 2 * G else 0
    if (batch.max_q_len != 1 or n != batch.n_seqs or hd % 16 or hd > 128 or H % G or H // G > 16
            or rot % 4 or rot > hd or width != (H + 2 * G) * hd or part.dtype != torch.float32
            or k_pages.dtype != torch.bfloat16 or table.shape[1] * 2 * 65 >= 1 << 31):
        return None
    require_device(part, k_pages, v_pages, table, batch.start_pos, *([freqs] if rot else []))
    require_contiguous(part=part, k_pages=k_pages, v_pages=v_pages, table=table)
    if tuple(k_pages.shape[1:]) != (G, 64, hd) or tuple(v_pages.shape[1:]) != (G, hd, 64):
        raise KernelError(f"attention_sliced: pages are {tuple(k_pages.shape)} / {tuple(v_pages.shape)}")
    if rot and (freqs.dtype != torch.float32 or freqs.numel() != rot // 2 or not freqs.is_contiguous()):
        raise KernelError("attention_sliced: one float32 frequency per rotated pair")
    if batch.start_pos.numel() != n or table.shape[0] < n or table.dtype != torch.int32:
        raise KernelError("attention_sliced: one position and one table row per sequence")
    rt, nw, tiles, splits = plan(n, 1, H, G, hd, table.shape[1])
    out = torch.empty((n, H, hd), dtype=torch.bfloat16, device=part.device)
    ws_o = ws_ml = None
    if splits > 1:
        ws_o = torch.empty((splits, n * H, hd), dtype=torch.float32, device=part.device)
        ws_ml = torch.empty((splits, n * H, 2), dtype=torch.float32, device=part.device)
    check(library("attention_bf16").gfa_attention_sliced_bf16(
        ptr(part), _i(S), ptr(freqs) if rot else None, _i(rot), ptr(k_pages), ptr(v_pages),
        _i(int(bool(write_cache))), ptr(batch.start_pos), ptr(table), _i(table.shape[1]), ptr(out),
        ptr(ws_o), ptr(ws_ml), _i(n), _i(H), _i(G), _i(hd), _f(scale), _i(window), _i(nw), _i(splits),
        stream_handle()), "attention_sliced_bf16")
    return out

