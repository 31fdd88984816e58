#!/usr/bin/env python3
"""Batched prompt pass of the full 36-layer model (awq_prefill_batched): milliseconds and tokens per second by
prompt length.  Synthetic balanced weights, cache capacity 40,960 positions, best of two runs per length.
Run on the GPU box: python cuda-kernel-qwen3-8b-awq_amd/bench_prefill.py [lengths, comma separated]
"""
import sys, os, time, ctypes, importlib
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
lib = awq.load_library()
lengths = [int(v) for v in sys.argv[1].split(",")] if len(sys.argv) > 1 else [32, 128, 256, 576, 1024, 1280, 2040,
                                                                             4096, 8192, 30000]
cfg = awq.make_config(n_layers=36, max_pos=40960)
eng = awq.QWen3AWQInfer.empty(cfg)
for layer, kind, part in awq.tensor_list(cfg):
    count = cfg.part_count(kind, part)
    nbytes = count if (part == awq.P_PACKED and kind != awq.T_GAMMA) else 2 * count
    buf = (ctypes.c_uint8 * nbytes)()
    awq.check(lib.awq_synth_fill_profile(awq.SYNTH_BALANCED, 1, layer, kind, part, buf, count))
    eng.upload(layer, kind, part, buf, nbytes)
eng.finalize()
for P in lengths:
    prompt = [(7 * i + 3) % 1000 for i in range(P)]
    best = 1e9
    for rep in range(2):
        eng.reset()
        t = time.perf_counter()
        eng.prefill(prompt, batched=True)   # returns after the device finished
        best = min(best, time.perf_counter() - t)
    print("prompt of %6d tokens: %8.1f ms  %7.0f tok/s" % (P, best * 1e3, P / best), flush=True)
eng.close()
