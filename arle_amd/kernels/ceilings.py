"""What one GPU gives to a kernel that only reads memory and to one that only multiplies on the matrix cores
(`csrc/ceilings.hip`): the measured ceilings that the engine's kernels are set against, beside the published
peaks.  No part of a model step."""
from __future__ import annotations

import ctypes
import time

import torch

from . import lib


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def read_bandwidth(device="cuda:0", total_bytes: int = 4 << 30, launches: int = 1, workgroups: int | None = None,
                   repeats: int = 5) -> dict:
    """Bytes a second of a read of `total_bytes` of HBM by workgroups that stay (best of `repeats`), as one launch
    or as `launches` launches in a row of an equal part each (what a kernel of that size can get at most)."""
    dev = torch.device(device)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    buf = torch.zeros(total_bytes, dtype=torch.uint8, device=dev)
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    part = total_bytes // launches // 4096 * 4096
    out = {}
    for wgs in ([workgroups] if workgroups else [cus, 2 * cus]):
        done = ctypes.c_longlong(0)
        best = float("inf")
        for _ in range(repeats + 1):
            torch.cuda.synchronize(dev)
            t = time.perf_counter()
            for i in range(launches):
                lib.call("arle_ceiling_read", buf.data_ptr() + i * part, part, wgs, ctypes.addressof(done), sink.data_ptr(),
                         _stream())
            torch.cuda.synchronize(dev)
            best = min(best, time.perf_counter() - t)
        out[wgs] = done.value * launches / best
    return {"bytes": total_bytes, "launches": launches, "by_workgroups": out, "best": max(out.values())}


def mfma_rate(device="cuda:0", shape: int = 32, iters: int = 20000, repeats: int = 3, random_operands: bool = True,
              workgroups: int | None = None) -> float:
    """Flops a second of waves that do nothing but bfloat16 matrix-core products (16 waves a compute unit, or
    `workgroups` of four waves over the chip).  `random_operands`: operands whose bits differ, as real data's do;
    the chip clocks lower under them than under operands that are all alike."""
    dev = torch.device(device)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    wgs = workgroups or cus * 4
    best = float("inf")
    for _ in range(repeats + 1):
        torch.cuda.synchronize(dev)
        t = time.perf_counter()
        lib.call("arle_ceiling_mfma", shape, iters, wgs, 1 if random_operands else 0, sink.data_ptr(), _stream())
        torch.cuda.synchronize(dev)
        best = min(best, time.perf_counter() - t)
    return wgs * 4 * iters * 262144.0 / best
