#!/usr/bin/env python3
"""Decode benchmark of the MI355X AWQ int4 engine.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one greedy decode step at batch 1 of the full Qwen3-8B-shaped model of the
reference (36 layers, hidden 4096, intermediate 12288, vocabulary 151936, int4 g=128; random-init
seeded weights, 128-token synthetic prompt).  Weights are resident in HBM before the timed region.
Prints ONE JSON line: decode tok/s, the HBM roofline of the dominant kernel (the fused int4
dequant + matrix-vector product, measured live with HIP events on the engine's stream) and the CPU
oracle timed on this host's cores on a bounded sample of the same workload.

Other modes (plain text output, used for the summaries under profiles/):
    --mode attention [--one-cache]   decode attention by attended length
    --mode prefill [--lengths a,b]   batched prompt pass of the 36-layer model by prompt length
    --mode traffic                   a 1 GiB copy, then the engine's w1 launches (for rocprofv3 --pmc runs)
    --mode w4a16                     W4A16 products of config 5 (token sweep on the w1 and w2 shapes)
"""
import argparse
import ctypes
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def mode_attention(args):
    """Decode attention (one query per head against the KV cache) at growing attended lengths:
    microseconds per launch and algorithmic GB/s (keys and values once: 2 x heads x L x 256 bytes).
    32 heads, caches of 40,960 positions with random binary16 contents, HIP events around the launches.
    Every launch reads another layer's cache (12 caches, 8 GB), as a decode step does: up to a few
    thousand positions one cache would stay in the L2 of each die (or the memory-side cache) between
    launches and flatter the short lengths; --one-cache shows that case."""
    import torch
    awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
    lib = awq.load_library()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    H, MP = 32, 40960
    NL = 1 if args.one_cache else 12
    kcs = [torch.randn(H, MP, 128, dtype=torch.float16, device="cuda") for _ in range(NL)]
    vcs = [torch.randn(H, MP, 128, dtype=torch.float16, device="cuda") for _ in range(NL)]
    q = torch.randn(H * 128, dtype=torch.float16, device="cuda")
    ctx = torch.empty(H * 128, dtype=torch.float16, device="cuda")
    ws = torch.zeros(lib.awq_attention_workspace_bytes(H, MP), dtype=torch.uint8, device="cuda")
    # a 1 GiB copy first: under `rocprofv3 --pmc FETCH_SIZE` its known size calibrates the counter's unit
    src = torch.full((1 << 28,), 1.0, dtype=torch.float32, device="cuda")
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst
    for L in [int(v) for v in args.att_lengths.split(",")]:
        def run(i):
            awq.check(lib.awq_decode_attention(q.data_ptr(), kcs[i % NL].data_ptr(), vcs[i % NL].data_ptr(),
                                               ctx.data_ptr(), H, MP, L, ws.data_ptr(), st))
        for i in range(NL):
            run(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n = 24
        e0.record()
        for i in range(n):
            run(i)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1000 / n
        nbytes = 2 * H * L * 128 * 2
        print("L=%6d  %9.1f us  %7.1f GB/s" % (L, us, nbytes / us / 1e3), flush=True)


def _synthetic_engine(awq, lib, cfg, seed, profile):
    eng = awq.QWen3AWQInfer.empty(cfg)
    for layer, kind, part in awq.tensor_list(cfg):
        count = cfg.part_count(kind, part)
        nbytes = count if (part == awq.P_PACKED and kind != awq.T_GAMMA) else 2 * count
        buf = (ctypes.c_uint8 * nbytes)()
        awq.check(lib.awq_synth_fill_profile(profile, seed, layer, kind, part, buf, count))
        eng.upload(layer, kind, part, buf, nbytes)
    eng.finalize()
    return eng


def mode_prefill(args):
    """Batched prompt pass of the full 36-layer model (awq_prefill_batched): milliseconds and tokens per
    second by prompt length.  Synthetic balanced weights, cache capacity 40,960 positions, best of two."""
    awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
    lib = awq.load_library()
    lengths = [int(v) for v in args.lengths.split(",")]
    eng = _synthetic_engine(awq, lib, awq.make_config(n_layers=36, max_pos=40960), 1, awq.SYNTH_BALANCED)
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


def mode_fused_timeline(args):
    """Where the time of the fused Wo + W1 launch goes (awq_set_fused_mode, off by default): the launch of every
    layer of the 36-layer model back to back, one of them instrumented -- thread 0 of each of its 256 workgroups
    notes the device time at 13 points.  Printed per point: minimum, median, 90th percentile and maximum over
    the workgroups, in microseconds after the first workgroup started.  Next to it the decode rate with one
    launch and with two."""
    import numpy as np
    import torch  # noqa: F401  (the HIP runtime of the process)
    awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
    lib = awq.load_library()
    eng = _synthetic_engine(awq, lib, awq.make_config(n_layers=36, max_pos=640), 1, awq.SYNTH_BALANCED)
    names = ["workgroup starts", "ctx, gamma, scales, Wo weights requested", "ctx arrived and staged (wavefront 0)",
             "... (all wavefronts)", "Wo multiplied (wavefront 0: its weights have arrived)", "... (all wavefronts)",
             "new hidden rows stored (tagged, device scope)", "whole new hidden state seen (wavefront 0)",
             "... (all wavefronts); W1 weights were requested after the store", "normalised and staged",
             "W1 multiplied (wavefront 0)", "... (all wavefronts)", "GeLU, stores, end"]
    for layer in (9, 27):
        buf = np.zeros(256 * 16, dtype=np.uint64)
        nw, ns = ctypes.c_int32(0), ctypes.c_int32(0)
        awq.check(lib.awq_debug_fused_timeline(eng._h, layer, buf.ctypes.data_as(ctypes.c_void_p), ctypes.byref(nw),
                                               ctypes.byref(ns)))
        t = buf[:nw.value * ns.value].reshape(nw.value, ns.value).astype(np.int64)
        us = (t - t[:, 0].min()) * 0.01
        print("fused Wo + W1 launch of layer %d, %d workgroups: microseconds after the first workgroup's start" %
              (layer, nw.value))
        print("  %-60s %7s %7s %7s %7s" % ("point", "min", "median", "p90", "max"))
        for k in range(ns.value):
            v = np.sort(us[:, k])
            print("  %-60s %7.2f %7.2f %7.2f %7.2f" % (names[k], v[0], v[len(v) // 2], v[len(v) * 9 // 10], v[-1]))
    prompt = [(7 * i + 3) % 1000 for i in range(128)]
    for fused in (False, True, False, True):
        eng.set_fused_mode(fused)
        eng.reset()
        eng.prefill(prompt, batched=True)
        eng.decode(8)
        t0 = time.perf_counter()
        eng.decode(256)
        dt = time.perf_counter() - t0
        print("decode, 256 steps after a 128-token prompt, Wo and W1 as %s: %.1f tok/s" %
              ("one launch " if fused else "two launches", 256 / dt), flush=True)
    eng.close()


def mode_qkv_timeline(args):
    """Where the time of the fused Wqkv + attention launch goes: the launch of every layer of the 36-layer model
    back to back, one of them instrumented -- thread 0 of each of its 256 workgroups notes the device time at 11
    points.  Printed per point: minimum, median, 90th percentile and maximum over the workgroups, in
    microseconds after the first workgroup started.  Next to it the decode rate with one launch and with two."""
    import numpy as np
    import torch  # noqa: F401  (the HIP runtime of the process)
    awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
    lib = awq.load_library()
    eng = _synthetic_engine(awq, lib, awq.make_config(n_layers=36, max_pos=768), 1, awq.SYNTH_BALANCED)
    names = ["workgroup starts", "x, gamma, state, scales, Q weights requested", "x normalised and staged (wavefront 0)",
             "... (all wavefronts); K and V weights and the cache rows requested now",
             "Q, K, V multiplied (wavefront 0: its weights have arrived)", "... (all wavefronts)",
             "this workgroup's Q, K, V rotated", "... and in LDS for all wavefronts (the cache appends follow)",
             "wavefront 0 past the partial scores (the streaming wavefronts publish theirs about now)",
             "all partial scores of the head seen, scores finished", "softmax, context of 16 dimensions, end"]
    for pos in (200, 600):
        for layer in (9, 27):
            buf = np.zeros(256 * 16, dtype=np.uint64)
            nw, ns = ctypes.c_int32(0), ctypes.c_int32(0)
            awq.check(lib.awq_debug_qkv_attention_timeline(eng._h, layer, pos, buf.ctypes.data_as(ctypes.c_void_p),
                                                           ctypes.byref(nw), ctypes.byref(ns)))
            t = buf[:nw.value * ns.value].reshape(nw.value, ns.value).astype(np.int64)
            us = (t - t[:, 0].min()) * 0.01
            print("fused Wqkv + attention launch of layer %d at position %d, %d workgroups: microseconds after the first "
                  "workgroup's start" % (layer, pos, nw.value))
            print("  %-72s %7s %7s %7s %7s" % ("point", "min", "median", "p90", "max"))
            for k in range(ns.value):
                v = np.sort(us[:, k])
                print("  %-72s %7.2f %7.2f %7.2f %7.2f" % (names[k], v[0], v[len(v) // 2], v[len(v) * 9 // 10], v[-1]))
    prompt = [(7 * i + 3) % 1000 for i in range(128)]
    for fused in (0, 2, 0, 2):
        eng.set_fused_mode(fused)
        eng.reset()
        eng.prefill(prompt, batched=True)
        eng.decode(8)
        t0 = time.perf_counter()
        eng.decode(256)
        dt = time.perf_counter() - t0
        print("decode, 256 steps after a 128-token prompt, Wqkv and attention as %s: %.1f tok/s" %
              ("one launch " if fused else "two launches", 256 / dt), flush=True)
    eng.close()


def mode_traffic(args):
    """Workload for the HBM-traffic counters of the decode GEMV kernel.  Run under
    `rocprofv3 --pmc FETCH_SIZE` and again under `rocprofv3 --pmc WRITE_SIZE`:
      1. a plain device-to-device copy of 1 GiB (reads 1 GiB, writes 1 GiB): the calibration of what
         the counters report per byte;
      2. the engine's own w1 launches (12288 x 4096 int4, RMSNorm prologue, GeLU epilogue) over the
         resident weights of a 12-layer model (302 MB of w1 matrices, above the last-level cache), 10 rounds.
    The per-dispatch counter values of the gemv kernel, scaled by the copy kernel's ratio of known
    bytes to counted units, give the HBM bytes per launch."""
    import torch
    awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
    src = torch.full((1 << 28,), 1.0, dtype=torch.float32, device="cuda")  # 1 GiB
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst
    eng = awq.QWen3AWQInfer.from_synthetic(awq.make_config(n_layers=12, max_pos=256), 11)
    us, nbytes = eng.time_linear(awq.T_W1, 10)
    print("w1 launch: %.2f us, %d algorithmic bytes" % (us, nbytes))
    eng.close()


def mode_w4a16(args):
    w4a16 = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd.bench_w4a16")
    tokens = tuple(int(v) for v in args.tokens.split(","))
    print(json.dumps(w4a16.measure(tokens, tuple(args.shapes.split(",")))), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=36, help="debug only: fewer layers make the result invalid")
    ap.add_argument("--prompt-len", type=int, default=128)
    ap.add_argument("--seed", type=int, default=2024)
    ap.add_argument("--max-pos", type=int, default=40960, help="positions the key/value cache is allocated for")
    ap.add_argument("--cpu-prompt", type=int, default=16, help="prompt length of the CPU sample")
    ap.add_argument("--cpu-steps", type=int, default=112, help="generated tokens of the CPU sample (0 = skip)")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-fused", action="store_true", help="one launch per product: no pair of a layer's launches runs as one")
    ap.add_argument("--fused", type=int, default=None,
                    help="which pairs of a layer's launches run as one: 1 Wo + W1, 2 Wqkv + attention, 3 both (default: the engine's)")
    ap.add_argument("--mode", choices=["decode", "steps", "attention", "prefill", "traffic", "w4a16", "fused-timeline", "qkv-timeline"], default="decode",
                    help="decode: the benchmark line; steps: only the prompt and the timed decode steps (for traces)")
    ap.add_argument("--one-cache", action="store_true", help="--mode attention: every launch reads the same cache")
    ap.add_argument("--att-lengths", default="128,256,512,576,577,768,1024,1025,1536,2048,2049,4096,8192,16384,40960",
                    help="--mode attention: attended lengths")
    ap.add_argument("--lengths", default="32,128,256,576,1024,1280,2040,4096,8192,30000", help="--mode prefill")
    ap.add_argument("--tokens", default="1,4,16,64,128,512,2048", help="--mode w4a16: token counts")
    ap.add_argument("--shapes", default="w1,w2", help="--mode w4a16: of w1 (12288x4096), w2 (4096x12288), wo (4096x4096)")
    ap.add_argument("--no-load-test", action="store_true",
                    help="skip writing the 3.64 GB weight directory and timing the loader on it")
    ap.add_argument("--no-spec-leg", action="store_true",
                    help="skip the second decode run on weights drawn from the benchmark definition's distributions")
    ap.add_argument("--profile", choices=["balanced", "spec"], default="balanced",
                    help="value distributions of the synthetic weights (include/awq_synth.h); 'spec' overflows "
                         "binary16 by layer 3 and decodes token 0 forever, so the default keeps activations finite")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs the whole model on ONE GPU (the reference's two-GPU layer split is "
              "collapsed onto one MI355X); --gpus %d is not supported, use --gpus 1" % args.gpus, file=sys.stderr)
        sys.exit(2)
    if args.mode == "steps":
        args.cpu_steps = 0
    if args.mode not in ("decode", "steps"):
        return {"attention": mode_attention, "prefill": mode_prefill, "traffic": mode_traffic,
                "fused-timeline": mode_fused_timeline, "qkv-timeline": mode_qkv_timeline,
                "w4a16": mode_w4a16}[args.mode](args)

    import numpy as np
    import torch
    awq = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")
    lib = awq.load_library()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from helpers import fill_pair, make_oracle_model, ptr
    import oracle_lib

    # the reference's sequence capacity (MAX_SEQ_LEN, Inference.cu:39): 24 GB of key/value cache
    cfg = awq.make_config(n_layers=args.layers, max_pos=args.max_pos)
    assert args.max_pos >= max(2176, args.prompt_len + args.warmup + args.steps + 8)
    oracle = oracle_lib.load() if args.cpu_steps > 0 else None

    profile = awq.SYNTH_BALANCED if args.profile == "balanced" else awq.SYNTH_SPEC
    t0 = time.time()
    eng = awq.QWen3AWQInfer.empty(cfg)
    if oracle is not None:
        # the checker owns the host copy of the weights; the engine gets the same bytes
        # (with room for its own sample only: its cache lives in host memory)
        model = make_oracle_model(oracle, awq.make_config(n_layers=args.layers, max_pos=args.cpu_prompt + args.cpu_steps + 8))
        fill_pair(awq, oracle, cfg, args.seed, engine=eng, model=model, profile=profile)
    else:
        model = None
        eng.close()
        eng = _synthetic_engine(awq, lib, cfg, args.seed, profile)
    eng.set_graph_mode(not args.no_graph)
    if args.no_fused:
        eng.set_fused_mode(0)
    elif args.fused is not None:
        eng.set_fused_mode(args.fused)
    eng_fused_mode = eng.fused_mode()
    log("fused launches (1 Wo + W1, 2 Wqkv + attention): %d" % eng_fused_mode)
    log("weights generated, uploaded and reordered in %.1f s" % (time.time() - t0))

    prompt = np.zeros(args.prompt_len, dtype=np.int32)
    awq.check(lib.awq_synth_tokens(args.seed, awq.SYNTH_STREAM_INPUT, ptr(prompt), prompt.size, cfg.vocab))

    if args.mode == "steps":
        eng.prefill(prompt.tolist(), batched=True)
        eng.decode(args.warmup)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        eng.decode(args.steps)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t1
        print(json.dumps({"mode": "steps", "prompt_len": args.prompt_len, "steps": args.steps,
                          "tok_s": round(args.steps / elapsed, 1), "ms_per_step": round(1e3 * elapsed / args.steps, 4)}))
        return

    # ---- the prompt pass, both ways (not part of `value`): token by token as the reference does,
    #      and all positions through each layer together on the matrix cores ---------------------
    prefill_ms = {}
    for name, batched in (("batched", True), ("sequential", False)):
        for rep in range(2):                       # the first pass builds graphs / allocates buffers
            eng.reset()
            torch.cuda.synchronize()
            tp = time.perf_counter()
            eng.prefill(prompt.tolist(), batched=batched)   # returns after the device finished
            prefill_ms[name] = round(1000.0 * (time.perf_counter() - tp), 3)
    log("prompt of %d tokens: %.2f ms token by token, %.2f ms batched" %
        (args.prompt_len, prefill_ms["sequential"], prefill_ms["batched"]))

    # ---- timed decode: K steps after the prompt and W warm-up steps ------------------------------
    eng.reset()
    eng.prefill(prompt.tolist())
    eng.decode(args.warmup)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    eng.decode(args.steps)          # returns after the device finished (stream synchronised inside)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t1
    tok_s = args.steps / elapsed
    ms_per_step = 1000.0 * elapsed / args.steps
    # attended length grows over the timed region; algorithmic bytes use its mean
    L_mean = args.prompt_len + args.warmup + (args.steps + 1) / 2.0
    per_layer = sum(cfg.part_count(k, awq.P_PACKED) for k in (awq.T_WQKV, awq.T_WO, awq.T_W1, awq.T_W2))
    weight_bytes = cfg.n_layers * per_layer + cfg.part_count(awq.T_UNEMBED, awq.P_PACKED)
    kv_bytes = cfg.n_layers * 2 * cfg.hidden * 2 * L_mean
    step_bytes = weight_bytes + kv_bytes
    log("decode: %.1f tok/s, %.3f ms/step, %.1f GB/s algorithmic (%.1f%% of 8 TB/s)" %
        (tok_s, ms_per_step, step_bytes / elapsed * args.steps / 1e9, 100 * step_bytes * tok_s / 8e12))

    # ---- roofline of the dominant kernel: fused int4 dequant + GEMV, w1 shape (12288 x 4096) -----
    kernels = {}
    for name, kind in (("w1", awq.T_W1), ("wqkv", awq.T_WQKV), ("w2", awq.T_W2), ("wo", awq.T_WO),
                       ("unembed", awq.T_UNEMBED)):
        us, nbytes = eng.time_linear(kind, 60 if kind != awq.T_UNEMBED else 200)
        kernels[name] = {"us": round(us, 3), "bytes": nbytes, "GBs": round(nbytes / us / 1e3, 1)}
        log("gemv %-8s %8.2f us/launch  %7.1f GB/s  (%.1f%% of peak)" % (name, us, nbytes / us / 1e3,
                                                                        nbytes / us / 1e3 / HBM_PEAK_GBS * 100))
    # the same launches on ONE layer's matrices (25 MB, resident in the last-level cache): the
    # cache-hot figure next to the rotating one above
    hot_cfg = awq.make_config(n_layers=1, max_pos=64)
    hot = _synthetic_engine(awq, lib, hot_cfg, args.seed, profile)
    for name, kind in (("w1", awq.T_W1), ("wqkv", awq.T_WQKV), ("w2", awq.T_W2), ("wo", awq.T_WO)):
        us, _ = hot.time_linear(kind, 400)
        kernels[name]["us_cache_hot"] = round(us, 3)
    hot.close()
    log("cache-hot (one layer's matrices): " + ", ".join("%s %.2f us" % (n, kernels[n]["us_cache_hot"])
                                                         for n in ("w1", "wqkv", "w2", "wo")))
    # HBM bytes per launch from the counter runs summarised under profiles/: only while the kernel's source is
    # the one they were measured on (the summary carries its SHA-256), null otherwise
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "gemv_w1_traffic.json")
    if os.path.exists(tpath):
        import hashlib
        rec = json.load(open(tpath))
        h = hashlib.sha256()
        for name in ("gemv.hip", "gemv_device.hpp"):  # the kernel and its device helpers
            src = os.path.join(ROOT, awq.__name__, "csrc", name)
            h.update(open(src, "rb").read() if os.path.exists(src) else b"missing")
        if h.hexdigest() == rec.get("gemv_sources_sha256"):
            traffic = rec.get("hbm_bytes_per_launch")
        else:
            log("profiles/gemv_w1_traffic.json was measured on another version of csrc/gemv.hip, "
                "csrc/gemv_device.hpp: traffic = null")
    w1 = kernels["w1"]
    roofline = {"bound": "hbm", "kernel": "gemv_kernel (int4 dequant + GEMV, m=12288 k=4096, GeLU epilogue)",
                "achieved": w1["GBs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(w1["GBs"] / HBM_PEAK_GBS, 4), "traffic": traffic,
                "bytes_per_launch": w1["bytes"], "us_per_launch": w1["us"], "all_shapes": kernels}

    # ---- one layer with about 512 cached positions (config 2): decode steps after a 512-token prompt,
    #      the unembedding's launch subtracted, divided by the layer count -------------------------
    p512 = np.zeros(512, dtype=np.int32)
    awq.check(lib.awq_synth_tokens(args.seed + 1, awq.SYNTH_STREAM_INPUT, ptr(p512), p512.size, cfg.vocab))
    eng.reset()
    eng.prefill(p512.tolist(), batched=True)
    eng.decode(8)
    torch.cuda.synchronize()
    t3 = time.perf_counter()
    eng.decode(64)
    torch.cuda.synchronize()
    step_us = (time.perf_counter() - t3) * 1e6 / 64
    layer_us = (step_us - kernels["unembed"]["us"]) / cfg.n_layers
    L_mid = 512 + 8 + 32
    layer_bytes = per_layer + 1024 + 8192 + 2 * cfg.hidden * 2 * L_mid + 16384
    layer_cfg2 = {"workload": "one layer (RMSNorm, Wqkv + rotary + KV append, attention, Wo, W1 + GeLU, W2), "
                              "attended length 520..584", "us": round(layer_us, 2), "bytes": int(layer_bytes),
                  "GBs": round(layer_bytes / layer_us / 1e3, 1),
                  "hbm_frac": round(layer_bytes / layer_us / 1e3 / HBM_PEAK_GBS, 4)}
    log("one layer at ~%d positions: %.1f us, %.0f GB/s (%.1f%% of peak)" %
        (L_mid, layer_us, layer_cfg2["GBs"], 100 * layer_cfg2["hbm_frac"]))

    # ---- the decode rate with a longer context: 64 steps after a batched 2040-token prompt (the
    #      attention takes three, then four launches cut along the sequence there) ---------------
    p2k = np.zeros(2040, dtype=np.int32)
    awq.check(lib.awq_synth_tokens(args.seed + 2, awq.SYNTH_STREAM_INPUT, ptr(p2k), p2k.size, cfg.vocab))
    eng.reset()
    torch.cuda.synchronize()
    t4 = time.perf_counter()
    eng.prefill(p2k.tolist(), batched=True)
    prompt_2k_ms = (time.perf_counter() - t4) * 1e3
    eng.decode(4)
    torch.cuda.synchronize()
    t5 = time.perf_counter()
    eng.decode(64)
    torch.cuda.synchronize()
    long_context = {"attended_positions": "2044..2108", "tok_s": round(64 / (time.perf_counter() - t5), 1),
                    "prompt_pass_ms_2040_tokens": round(prompt_2k_ms, 2)}
    log("decode at ~2k positions: %.1f tok/s; 2040-token prompt %.1f ms" % (long_context["tok_s"], prompt_2k_ms))

    # ---- the prompt pass's product on the matrix cores: w1 shape, 2048 tokens (config 5) ---------
    w4a16 = importlib.import_module("cuda-kernel-qwen3-8b-awq_amd.bench_w4a16")
    sweep = w4a16.measure((4, 16, 64, 2048), ("w1",))["shapes"]["w1"]
    g = sweep["M=2048"]
    # config 5's decode-batch points on the same matrix: a weight stream, priced against the HBM peak
    batch_gemm = {"workload": "W4A16 product 12288 x 4096 (int4 g=128) x 4 / 16 / 64 tokens, 12 rotating matrices",
                  "bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s",
                  "tokens": {str(M): {"us_per_launch": sweep["M=%d" % M]["us"], "achieved": sweep["M=%d" % M]["GBs"],
                                      "frac": sweep["M=%d" % M]["hbm_frac"]} for M in (4, 16, 64)}}
    prefill_gemm = {"workload": "W4A16 product 12288 x 4096 (int4 g=128) x 2048 tokens, 12 rotating matrices",
                    "bound": "mfma", "achieved": g["TFLOPs"], "peak": 2500.0, "unit": "TFLOP/s",
                    "frac": g["mfma_frac"], "us_per_launch": g["us"]}
    log("gemm w1 x 2048 tokens: %.1f us, %.0f TFLOP/s (%.1f%% of 2.5 PFLOP/s)" % (g["us"], g["TFLOPs"], 100 * g["mfma_frac"]))

    # ---- the same decode run on weights drawn from the benchmark definition's own distributions (scale
    #      U[0.002,0.02], zero-point 0..15): activations overflow binary16 within four layers and every id
    #      is 0, so it proves nothing about the arithmetic, but it shows that the rate does not depend on
    #      the values -----------------------------------------------------------------------------------
    spec_leg = None
    if not args.no_spec_leg and args.profile == "balanced":
        t6 = time.time()
        spec = _synthetic_engine(awq, lib, cfg, args.seed, awq.SYNTH_SPEC)
        spec.set_graph_mode(not args.no_graph)
        spec.prefill(prompt.tolist())
        spec.decode(args.warmup)
        torch.cuda.synchronize()
        t7 = time.perf_counter()
        spec_ids = spec.decode(args.steps)
        torch.cuda.synchronize()
        spec_elapsed = time.perf_counter() - t7
        spec.close()
        spec_leg = {"value": round(args.steps / spec_elapsed, 2), "unit": "tok/s",
                    "ms_per_step": round(1000.0 * spec_elapsed / args.steps, 4),
                    "data": "scale U[0.002,0.02], zero-point 0..15 (benchmark definition): activations overflow "
                            "binary16, distinct ids in the run: %d" % len(set(spec_ids))}
        log("decode on the benchmark definition's distributions: %.1f tok/s (engine built in %.1f s)" %
            (spec_leg["value"], time.time() - t6))

    # ---- the loader on a weight directory in the reference's layout (474 files, 3.64 GB), written just
    #      before: once with the files dropped from the page cache, once from the page cache ---------------
    load = None
    if not args.no_load_test and args.layers == 36:
        import shutil
        import tempfile
        d = tempfile.mkdtemp(prefix="awq_weights_")
        try:
            t8 = time.time()
            awq.check(lib.awq_write_weight_dir_profile(d.encode(), ctypes.byref(cfg), args.seed, profile))
            nbytes = sum(os.path.getsize(os.path.join(d, f)) for f in os.listdir(d))
            log("weight directory written in %.1f s (%d bytes)" % (time.time() - t8, nbytes))
            # cold: the files' pages are written back and dropped from the page cache first (fsync, then
            # POSIX_FADV_DONTNEED per file), so the reader thread gets them from the box's storage;
            # warm: the same directory again, now cached by that first pass
            dropped = 0
            for f in os.listdir(d):
                fd = os.open(os.path.join(d, f), os.O_RDONLY)
                try:
                    os.fsync(fd)
                    os.posix_fadvise(fd, 0, 0, os.POSIX_FADV_DONTNEED)
                    dropped += 1
                finally:
                    os.close(fd)
            legs = {}
            for leg in ("cold", "warm"):
                t9 = time.perf_counter()
                loaded = awq.QWen3AWQInfer(d, config=awq.make_config(n_layers=args.layers, max_pos=2176))
                create_s = time.perf_counter() - t9
                legs[leg] = (lib.awq_last_load_seconds(), create_s)
                loaded.close()
            load = {"load_s": round(legs["warm"][0], 3), "create_s": round(legs["warm"][1], 3),
                    "load_s_cold": round(legs["cold"][0], 3), "create_s_cold": round(legs["cold"][1], 3),
                    "bytes": nbytes, "GBs": round(nbytes / legs["warm"][0] / 1e9, 2),
                    "GBs_cold": round(nbytes / legs["cold"][0] / 1e9, 2),
                    "what": "load_s: first file opened to last tensor reordered on the device (reader thread, two "
                            "pinned buffers, copies and reordering overlapped); create_s: the whole awq_create with "
                            "allocation, rotary tables and a zeroed 2176-position cache.  *_cold: right after the "
                            "%d files were synced and dropped from the page cache (posix_fadvise DONTNEED); the "
                            "others: the same directory again, from the page cache" % dropped}
            log("loader: cold %.2f s (%.1f GB/s), warm %.2f s for %.2f GB (%.1f GB/s), whole constructor %.2f s" %
                (legs["cold"][0], load["GBs_cold"], load["load_s"], nbytes / 1e9, load["GBs"], legs["warm"][1]))
        finally:
            shutil.rmtree(d, ignore_errors=True)

    # ---- CPU oracle on this host's cores, bounded sample; and token identity on that sample ------
    cpu = None
    tokens_match = None
    if oracle is not None:
        cp = prompt[:args.cpu_prompt].copy()
        out = np.zeros(max(1, args.cpu_steps), dtype=np.int32)
        t2 = time.perf_counter()
        rc = oracle.awqo_model_generate(model, ptr(cp), cp.size, args.cpu_steps, ptr(out))
        cpu_s = time.perf_counter() - t2
        assert rc == args.cpu_steps
        passes = cp.size + args.cpu_steps
        gpu_tokens = eng.generateResponse(cp.tolist(), args.cpu_steps)
        tokens_match = "%d/%d" % (sum(int(a == b) for a, b in zip(gpu_tokens, out.tolist())), args.cpu_steps)
        cpu = {"value": round(passes / cpu_s, 3), "unit": "tok/s", "cores": oracle.awqo_num_threads(), "kind": "port",
               "sample": "%d-token prompt + %d greedy tokens = %d forward passes of the same 36-layer model, "
                         "%.1f s" % (cp.size, args.cpu_steps, passes, cpu_s)}
        log("cpu oracle: %.2f tok/s on %d threads; greedy tokens identical: %s" %
            (cpu["value"], cpu["cores"], tokens_match))

    line = {
        "metric": "decode tok/s @bs1, 8B-shape AWQ; int4 GEMV achieved HBM GB/s vs peak",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 weights; f16 activations held as 16-bit block fixed point per 32 inputs; exact integer block "
                 "products (int8 matrix cores on byte planes, 4-bit dot products for w2); f32 per-block scaling and "
                 "accumulation; f16 outputs",
        "data": "synthetic (seeded random-init; nibbles uniform 0..15; %s)" % (
            "value: scale U[0.0025,0.004], zero-point 7 or 8 so that activations stay finite; value_spec_profile: the "
            "benchmark definition's scale U[0.002,0.02], zero-point 0..15, whose activations overflow FP16"
            if args.profile == "balanced"
            else "scale U[0.002,0.02], zero-point 0..15 as in the benchmark definition: activations overflow FP16"),
        "config": {"workload": "full Qwen3-8B-shaped random-init AWQ model on one GPU: %d layers, hidden 4096, "
                               "intermediate 12288, vocab 151936, int4 g=128; %d-token prompt, batch-1 greedy decode"
                               % (cfg.n_layers, args.prompt_len),
                   "attended_positions": "%d..%d" % (args.prompt_len + args.warmup, args.prompt_len + args.warmup + args.steps),
                   "max_pos": cfg.max_pos, "graph": not args.no_graph,
                   "steps_per_graph_launch": 1 if args.no_graph else 4, "fused_launches": eng_fused_mode},
        "step_algorithmic_bytes": int(step_bytes),
        "step_hbm_frac": round(step_bytes * tok_s / (HBM_PEAK_GBS * 1e9), 4),
        "greedy_tokens_identical_to_cpu": tokens_match,
        "value_spec_profile": spec_leg,
        "loader": load,
        "prompt_pass_ms": prefill_ms,
        "layer_512_positions": layer_cfg2,
        "long_context": long_context,
        "prefill_gemm": prefill_gemm,
        "batch_gemm": batch_gemm,
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    eng.close()
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
