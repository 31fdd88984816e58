#!/usr/bin/env python3
"""Decode attention (one query per head against the KV cache) at growing attended lengths:
microseconds per launch and algorithmic GB/s (keys and values once: 2 x heads x L x 256 bytes).
32 heads, a cache of 40,960 positions with random binary16 contents, HIP events around 20 launches.
Run on the GPU box: python cuda-kernel-qwen3-8b-awq_amd/bench_attention.py
"""
import sys, os, ctypes, importlib
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import torch
awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
lib = awq.load_library()
st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
H, MP = 32, 40960
kc = torch.randn(H, MP, 128, dtype=torch.float16, device="cuda")
vc = torch.randn(H, MP, 128, dtype=torch.float16, device="cuda")
q = torch.randn(H * 128, dtype=torch.float16, device="cuda")
ctx = torch.empty(H * 128, dtype=torch.float16, device="cuda")
ws = torch.zeros(lib.awq_attention_workspace_bytes(H, MP), dtype=torch.uint8, device="cuda")
for L in (128, 256, 512, 768, 1024, 1536, 1792, 2000, 2048, 4096, 8192, 16384, 40960):
    def run():
        awq.check(lib.awq_decode_attention(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), ctx.data_ptr(), H, MP, L, ws.data_ptr(), st))
    for _ in range(3): run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20): run()
    e1.record(); torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1000 / 20
    nbytes = 2 * H * L * 128 * 2
    print("L=%6d  %9.1f us  %7.1f GB/s" % (L, us, nbytes / us / 1e3), flush=True)
