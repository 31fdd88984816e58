#!/usr/bin/env python3
"""Prefill / batched W4A16 products on the w1 and w2 shapes of the reference model
(w1 12288 x 4096, w2 4096 x 12288, int4 g=128, seeded weights):

  * M = 2048 tokens through the dequant-on-load MFMA kernel: TFLOP/s and the fraction of the
    MI355X dense FP16 matrix peak (2.5 PFLOP/s);
  * M = 1 through the decode kernel, M = 4, 16, 64, 128, 512 through the MFMA kernels: microseconds,
    algorithmic GB/s and the fraction of the 8 TB/s HBM peak.

An optional argument lists the token counts to run, e.g. 128,2048; a second one the shapes (w1,w2,wo;
wo is the 4096 x 4096 attention output matrix).

Weights rotate over several distinct matrices so that they come from HBM, not from cache.
Prints one JSON object.  Run on the GPU box: python bench.py --mode w4a16 [--tokens 128,2048] [--shapes w1,w2,wo]
"""
import ctypes
import importlib
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


ALL_SHAPES = (("w1", (12288, 4096)), ("w2", (4096, 12288)), ("wo", (4096, 4096)))


def measure(tokens, shapes=("w1", "w2")):
    """Time the products for the given token counts on the named shapes; returns the result dictionary."""
    import numpy as np
    import torch
    awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
    lib = awq.load_library()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {"mfma_peak_tflops": 2500.0, "hbm_peak_gbs": 8000.0, "shapes": {}}
    n_mat = 12  # 12 x 25 MB = 300 MB working set, above the 256 MB last-level cache
    for name, (m, k) in ALL_SHAPES:
        if name not in shapes:
            continue
        mats = []
        for i in range(n_mat):
            host = np.zeros(m * k // 2, dtype=np.uint8)
            awq.check(lib.awq_synth_fill(7, i, awq.T_W1 if name == "w1" else awq.T_W2, awq.P_PACKED,
                                         host.ctypes.data_as(ctypes.c_void_p), host.size))
            d_in = torch.from_numpy(host).cuda()
            d_w = torch.empty_like(d_in)
            awq.check(lib.awq_linear_repack(d_in.data_ptr(), d_w.data_ptr(), m, k, st))
            mats.append(d_w)
        torch.cuda.synchronize()
        sc = np.zeros(m // 128, dtype=np.float16)
        zp = np.zeros(m // 128, dtype=np.float16)
        awq.check(lib.awq_synth_fill(7, 0, awq.T_W1, awq.P_SCALE, sc.ctypes.data_as(ctypes.c_void_p), sc.size))
        awq.check(lib.awq_synth_fill(7, 0, awq.T_W1, awq.P_ZP, zp.ctypes.data_as(ctypes.c_void_p), zp.size))
        d_s, d_z = torch.from_numpy(sc).cuda(), torch.from_numpy(zp).cuda()
        ws = torch.zeros(lib.awq_gemv_workspace_bytes(m, k), dtype=torch.uint8, device="cuda")
        res = {}
        for M in tokens:
            x = torch.randn(M, k, dtype=torch.float16, device="cuda")
            y = torch.empty(M, m, dtype=torch.float16, device="cuda")
            gws = torch.zeros(max(16, lib.awq_gemm_workspace_bytes(m, k, M)), dtype=torch.uint8, device="cuda")

            def launch(i):
                w = mats[i % n_mat]
                if M == 1:
                    awq.check(lib.awq_gemv(w.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), m, k, x.data_ptr(),
                                           y.data_ptr(), ws.data_ptr(), st))
                else:
                    awq.check(lib.awq_gemm(w.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), m, k, x.data_ptr(),
                                           y.data_ptr(), M, 1, gws.data_ptr(), st))
            iters = 48 if M >= 512 else 120
            # warm-up by time, not by count: after an idle stretch (the host generating matrices) the
            # device needs some tens of milliseconds of work before its clocks are back up; a timing
            # taken right after 12 launches reads up to 20 % slow
            import time
            t_warm = time.perf_counter()
            while time.perf_counter() - t_warm < 0.06:
                for i in range(n_mat):
                    launch(i)
                torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(iters):
                launch(i)
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1000.0 / iters
            flops = 2.0 * m * k * M
            nbytes = m * k // 2 + 4 * (m // 128) + 2 * M * k + 2 * M * m
            res["M=%d" % M] = {"us": round(us, 2), "TFLOPs": round(flops / us / 1e6, 2),
                               "mfma_frac": round(flops / us / 1e6 / 2500.0, 4), "GBs": round(nbytes / us / 1e3, 1),
                               "hbm_frac": round(nbytes / us / 1e3 / 8000.0, 4),
                               "kernel": "gemv (VALU, bit-exact order)" if M == 1 else
                                         ("gemm (MFMA 16x16x32 f16)" if M <= 4 else "gemm (MFMA 32x32x16 f16)")}
            print(name, "M=%d" % M, res["M=%d" % M], file=sys.stderr, flush=True)
        out["shapes"][name] = res
        del mats
        torch.cuda.empty_cache()
    return out


def main():
    tokens = (1, 4, 16, 64, 128, 512, 2048)
    if len(sys.argv) > 1:
        tokens = tuple(int(v) for v in sys.argv[1].split(","))
    shapes = tuple(sys.argv[2].split(",")) if len(sys.argv) > 2 else ("w1", "w2")
    print(json.dumps(measure(tokens, shapes)))


if __name__ == "__main__":
    main()
