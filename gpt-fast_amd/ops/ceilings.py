"""What this GPU reaches with kernels that only stream memory or only issue matrix
instructions (csrc/ceilings.hip): the measured counterparts of the datasheet peaks that
a step's bandwidth and flops are compared with."""
import ctypes
import time

import torch

from .library import check, library, ptr, stream_handle

_i = ctypes.c_int
_sz = ctypes.c_size_t


def _timed(fn, repeats: int) -> float:
    fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(repeats):
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        best = min(best, time.perf_counter() - t0)
    return best


def measure(device="cuda:0", megabytes: int = 2048, repeats: int = 5) -> dict:
    """{"hbm_read_gbs", "hbm_copy_gbs", "mfma_bf16_tflops"}: best of ``repeats`` runs of a
    read of ``megabytes`` (far beyond the caches), a copy of it (bytes read + written), and
    a matrix-instruction loop on every compute unit."""
    lib = library("ceilings")
    n = megabytes * (1 << 20)
    src = torch.empty(n, dtype=torch.uint8, device=device).random_(0, 255)
    dst = torch.empty_like(src)
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    blocks = cus * 8
    sink = torch.zeros(blocks, dtype=torch.int32, device=device)
    s = stream_handle()
    t_read = _timed(lambda: check(lib.gfa_read_stream(ptr(src), _sz(n), ptr(sink), _i(blocks), s),
                                  "read_stream"), repeats)
    t_copy = _timed(lambda: check(lib.gfa_copy_stream(ptr(dst), ptr(src), _sz(n), _i(blocks), s),
                                  "copy_stream"), repeats)
    iters = 20000
    out = torch.empty(blocks * 256, dtype=torch.float32, device=device)
    t_mfma = _timed(lambda: check(lib.gfa_mfma_peak(ptr(out), _i(blocks), _i(iters), s),
                                  "mfma_peak"), repeats)
    flops = blocks * 4 * iters * 8 * 16 * 16 * 32 * 2
    return {"hbm_read_gbs": round(n / t_read / 1e9, 1),
            "hbm_copy_gbs": round(2 * n / t_copy / 1e9, 1),
            "mfma_bf16_tflops": round(flops / t_mfma / 1e12, 1)}
