#!/usr/bin/env python3
"""Decode attention (one query per head against the KV cache) at growing attended lengths:
microseconds per launch and algorithmic GB/s (keys and values once: 2 x heads x L x 256 bytes).
32 heads, caches of 40,960 positions with random binary16 contents, HIP events around the launches.
Every launch reads another layer's cache (12 caches, 8 GB), as a decode step does: up to a few thousand
positions one cache would stay in the 4 MB L2 of each die (or the 256 MB memory-side cache) between
launches and flatter the short lengths.  `--one-cache` shows that case.
Run on the GPU box: python cuda-kernel-qwen3-8b-awq_amd/bench_attention.py [--one-cache]
"""
import sys, os, ctypes, importlib
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import torch
awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
lib = awq.load_library()
st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
H, MP = 32, 40960
NL = 1 if "--one-cache" in sys.argv else 12
kcs = [torch.randn(H, MP, 128, dtype=torch.float16, device="cuda") for _ in range(NL)]
vcs = [torch.randn(H, MP, 128, dtype=torch.float16, device="cuda") for _ in range(NL)]
q = torch.randn(H * 128, dtype=torch.float16, device="cuda")
ctx = torch.empty(H * 128, dtype=torch.float16, device="cuda")
ws = torch.zeros(lib.awq_attention_workspace_bytes(H, MP), dtype=torch.uint8, device="cuda")
for L in (128, 256, 512, 576, 577, 768, 1024, 1025, 1536, 2048, 2049, 4096, 8192, 16384, 40960):
    def run(i):
        awq.check(lib.awq_decode_attention(q.data_ptr(), kcs[i % NL].data_ptr(), vcs[i % NL].data_ptr(), ctx.data_ptr(),
                                           H, MP, L, ws.data_ptr(), st))
    for i in range(NL): run(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n = 24
    e0.record()
    for i in range(n): run(i)
    e1.record(); torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1000 / n
    nbytes = 2 * H * L * 128 * 2
    print("L=%6d  %9.1f us  %7.1f GB/s" % (L, us, nbytes / us / 1e3), flush=True)
