"""What this GPU delivers, measured: the streaming read of cold memory and the matrix cores' rate.

A benchmark states its fractions of the published peaks (HBM 8 TB/s, 2.5 PFLOP/s of dense bfloat16), which no
kernel reaches, and beside them the fractions of what ``csrc/machine_peaks.hip`` reaches on the same machine in
the same process: a kernel that does nothing but read memory no cache holds, and one that does nothing but
issue matrix instructions on registers. The reference's report has no such figures (it publishes no numbers).
"""

from __future__ import annotations

from typing import Dict

import torch

from .. import kernels


def _best_ms(launch, repeats: int) -> float:
    launch()                                   # warm-up (and the library's first load)
    torch.cuda.synchronize()
    best = None
    for _ in range(repeats):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        launch()
        end.record()
        end.synchronize()
        ms = start.elapsed_time(end)
        best = ms if best is None else min(best, ms)
    return best


def measured_peaks(device="cuda:0", stream_bytes: int = 4 << 30, repeats: int = 5) -> Dict[str, float]:
    """``{"hbm_read_gbs": ..., "mfma_bf16_tflops": ...}``: the best of ``repeats`` runs of each kernel.

    The read goes over ``stream_bytes`` (far more than the 256 MB of the last-level cache, so every run finds
    its data in memory), from 2048 workgroups of four waves with 8 KB in flight a wave."""
    with torch.cuda.device(device):
        data = torch.empty(stream_bytes // 4, dtype=torch.int32, device=device)
        data.fill_(0x01020304)
        sink = torch.zeros(4, dtype=torch.int32, device=device)
        read = [0]

        def read_once():
            read[0] = kernels.stream_read(data, sink)

        ms = _best_ms(read_once, repeats)
        hbm = read[0] / (ms * 1e-3) / 1e9
        del data
        torch.cuda.empty_cache()
        fsink = torch.zeros(4, dtype=torch.float32, device=device)
        flops = [0.0]

        def multiply_once():
            flops[0] = kernels.mfma_rate(fsink)

        ms = _best_ms(multiply_once, repeats)
        return {"hbm_read_gbs": hbm, "mfma_bf16_tflops": flops[0] / (ms * 1e-3) / 1e12}
