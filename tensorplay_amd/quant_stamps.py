"""Where the time of the row quantizer goes: ``python -m tensorplay_amd.quant_stamps [rows] [K]``.

Runs the measuring build of the quantizer (libtpq_quant_stamps.so, built by build.py with -DTPQ_QUANT_STAMPS: the
register-cached kernel with six readings of the shader clock per workgroup) on bfloat16 rows, and prints
the length of each phase inside a workgroup, and from the chip-wide 100 MHz clock when workgroups enter and end.
The shipped library carries no stamps.
"""
import ctypes
import os
import sys

import numpy as np
import torch

from . import build

PHASES = ["entry", "loads issued", "own data reduced", "row maximum known", "stores issued", "stores acknowledged"]


def main(rows: int = 2048, k: int = 4096, repeats: int = 5, train: int = 20) -> None:
    if not os.path.exists(build.QUANT_STAMPS_LIB_PATH):
        raise RuntimeError("libtpq_quant_stamps.so is not built: run python -m tensorplay_amd.build")
    lib = ctypes.CDLL(build.QUANT_STAMPS_LIB_PATH)
    lib.tpq_last_error.restype = ctypes.c_char_p
    dev = torch.device("cuda:0")
    x = torch.randn(rows, k, device=dev).to(torch.bfloat16)
    codes = torch.empty((rows, k), dtype=torch.int8, device=dev)
    scales = torch.empty(rows, dtype=torch.float32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def launch():
        rc = lib.tpq_quantize_rowwise(ctypes.c_void_p(x.data_ptr()), 2, ctypes.c_int64(rows), ctypes.c_int64(k), ctypes.c_float(1e-5),
                                      ctypes.c_float(127.0), -127, 127, 0, ctypes.c_void_p(codes.data_ptr()),
                                      ctypes.c_void_p(scales.data_ptr()), stream)
        if rc != 0:
            raise RuntimeError(lib.tpq_last_error().decode())

    for _ in range(3):
        launch()
    torch.cuda.synchronize()
    n = min(rows, 8192)
    table = np.zeros((repeats, n, 8), dtype=np.uint64)
    times = []
    for r in range(repeats):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(train - 1):   # the stamps that remain are those of the last launch of a train: a warm chip
            launch()
        a.record()
        launch()
        b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b) * 1000)
        rc = lib.tpq_quantize_stamps_read(table[r].ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(n))
        if rc != 0:
            raise RuntimeError(lib.tpq_last_error().decode())
    t = table[:, :, :6].astype(np.int64)
    wall = table[:, :, 6:8].astype(np.int64)          # 100 MHz, one counter for the chip
    wall -= wall[:, :, 0].min(axis=1)[:, None, None]
    print(f"row quantizer {rows} x {k} bfloat16, the last of {train} launches back to back, {repeats} times: {np.median(times):.2f} us between events around it (median)")
    print("phase lengths inside a workgroup, shader clocks (the counters of different compute units share no zero)")
    print(f"{'phase':<40}{'median':>8}{'p95':>8}{'max':>8}")
    for i in range(1, 6):
        d = (t[:, :, i] - t[:, :, i - 1]).reshape(-1)
        print(f"{PHASES[i - 1] + ' -> ' + PHASES[i]:<40}{int(np.median(d)):>8d}{int(np.percentile(d, 95)):>8d}{d.max():>8d}")
    life = (t[:, :, 5] - t[:, :, 0]).reshape(-1)
    print(f"{'entry -> stores acknowledged':<40}{int(np.median(life)):>8d}{int(np.percentile(life, 95)):>8d}{life.max():>8d}")
    print("when workgroups enter and end, us since the first one entered (chip-wide 100 MHz clock, 0.01 us steps)")
    print(f"{'':<10}{'first':>8}{'median':>8}{'p95':>8}{'last':>8}")
    for i, name in enumerate(("entry", "end")):
        col = wall[:, :, i].reshape(-1) / 100.0
        print(f"{name:<10}{col.min():>8.2f}{np.median(col):>8.2f}{np.percentile(col, 95):>8.2f}{col.max():>8.2f}")
    span = (wall[:, :, 1] - wall[:, :, 0]).reshape(-1) / 100.0
    print(f"a workgroup lives {np.median(span):.2f} us (median), {span.max():.2f} at most")


if __name__ == "__main__":
    args = [int(a) for a in sys.argv[1:3]]
    main(*args)
