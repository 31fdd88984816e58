#!/usr/bin/env python3
"""Workload for the HBM-traffic counters of the decode GEMV kernel.

Run under `rocprofv3 --pmc FETCH_SIZE` and again under `rocprofv3 --pmc WRITE_SIZE`:
  1. a plain device-to-device copy of 1 GiB (reads 1 GiB, writes 1 GiB) -- the calibration of
     what the counters report per byte;
  2. the engine's own w1 launches (12288 x 4096 int4, RMSNorm prologue, GeLU epilogue) over the
     resident weights of an 8-layer model, 10 rounds.
The per-dispatch counter values of the gemv kernel, scaled by the copy kernel's ratio of
known bytes to counted units, give the HBM bytes per launch.
"""
import ctypes
import importlib
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def main():
    import torch
    awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
    src = torch.full((1 << 28,), 1.0, dtype=torch.float32, device="cuda")  # 1 GiB
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst
    cfg = awq.make_config(n_layers=12, max_pos=256)  # 12 distinct w1 matrices = 302 MB, above the last-level cache
    eng = awq.QWen3AWQInfer.from_synthetic(cfg, 11)
    us, nbytes = eng.time_linear(awq.T_W1, 10)
    print("w1 launch: %.2f us, %d algorithmic bytes" % (us, nbytes))
    eng.close()


if __name__ == "__main__":
    main()
