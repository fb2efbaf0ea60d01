"""What the machine delivers, measured: streaming reads from HBM and matrix-core arithmetic on
random data.  Used by the measurement script beside the published peaks; not part of the model's
path."""
from __future__ import annotations

import torch

from . import kernels, library
from .kernels import _I, _L, _P

kernels.register_signatures("peaks", {
    "agave_peak_read": [_P, _L, _P, _I, _P],
    "agave_peak_mfma": [_P, _P, _I, _I, _P],
})


def _timed(fn, repeats: int) -> float:
    """Seconds per call, from a pair of events around ``repeats`` calls (after one warm-up)."""
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(repeats):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / repeats


def hbm_read_gbs(device="cuda:0", gib: int = 2, workgroups: int = 2048) -> float:
    """GB/s of a kernel that reads ``gib`` GiB once (far more than the caches hold)."""
    buf = torch.empty(gib << 30, dtype=torch.uint8, device=device)
    buf.fill_(1)
    sink = torch.zeros(1, dtype=torch.int32, device=device)
    lib = kernels.lib("peaks")
    dt = _timed(lambda: library.call(lib, "agave_peak_read", buf.data_ptr(), buf.numel(), sink.data_ptr(), workgroups,
                                     kernels.stream()), 5)
    return buf.numel() / dt / 1e9


def mfma_bf16_tflops(device="cuda:0", workgroups: int = 256, iters: int = 20000) -> float:
    """TFLOP/s of a loop of 32x32x16 bfloat16 matrix-core instructions on N(0, 1) operands, one
    workgroup of eight waves per compute unit."""
    g = torch.Generator(device=device).manual_seed(0)
    src = torch.randn(6 * 512 * 8, generator=g, device=device).bfloat16()
    out = torch.empty(workgroups * 512, dtype=torch.float32, device=device)
    lib = kernels.lib("peaks")
    dt = _timed(lambda: library.call(lib, "agave_peak_mfma", src.data_ptr(), out.data_ptr(), workgroups, iters,
                                     kernels.stream()), 2)
    return 2.0 * 32 * 32 * 16 * 8 * iters * 8 * workgroups / dt / 1e12
