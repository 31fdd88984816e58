"""CPU-side checks of the drop-in boundary: the shared library loads without a GPU, exports every
symbol that include/awq_infer.h declares, validates weight directories before touching HIP, and the
seeded generator agrees with an independent numpy statement and with the committed fixture."""
import ctypes
import json
import os
import re
import subprocess

import numpy as np
import pytest

import helpers
from helpers import ptr

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "awq_infer.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(awq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(awq, lib):
    names = declared_functions()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), n
        assert n in awq.SIGNATURES, "binding missing for " + n
    assert set(awq.SIGNATURES) == set(names)


def test_default_config_is_the_reference(awq):
    c = awq.default_config()
    assert (c.n_layers, c.hidden, c.inter, c.vocab, c.max_pos, c.split_idx) == (36, 4096, 12288, 151936, 40960, 18)
    assert abs(c.eps - 1e-6) < 1e-12


def test_weight_file_table_matches_reference_sizes(awq, lib, tmp_path):
    """write the directory for a small shape and check names and sizes follow Inference.cu:780-899;
    the full-size byte counts are checked arithmetically"""
    cfg = awq.make_config(n_layers=2, hidden=512, inter=1024, vocab=1280, max_pos=16)
    d = str(tmp_path)
    awq.check(lib.awq_write_weight_dir(d.encode(), ctypes.byref(cfg), 5))
    files = sorted(os.listdir(d))
    assert len(files) == 2 * 13 + 6
    assert os.path.getsize(os.path.join(d, "layer_1_w1.bin")) == 1024 * 512 // 2
    assert os.path.getsize(os.path.join(d, "layer_1_w2_scale.bin")) == (512 // 128) * 2
    assert os.path.getsize(os.path.join(d, "word_embedding.bin")) == 512 * 1280 // 2
    assert os.path.getsize(os.path.join(d, "word_embed_zp.bin")) == (512 // 128) * 2
    assert os.path.getsize(os.path.join(d, "unembed_scale.bin")) == (1280 // 128) * 2
    assert lib.awq_validate_weight_dir(d.encode(), ctypes.byref(cfg)) == 0
    # contents are the seeded stream
    got = np.fromfile(os.path.join(d, "layer_1_wo.bin"), dtype=np.uint8)
    assert np.array_equal(got, helpers.synth_packed(5, 1, awq.T_WO, got.size))
    # missing file
    os.remove(os.path.join(d, "rms_norm_gamma_0.bin"))
    assert lib.awq_validate_weight_dir(d.encode(), ctypes.byref(cfg)) == 2
    assert b"could not open" in lib.awq_last_error() and b"rms_norm_gamma_0.bin" in lib.awq_last_error()
    # short file
    open(os.path.join(d, "rms_norm_gamma_0.bin"), "wb").write(b"\0" * 10)
    assert lib.awq_validate_weight_dir(d.encode(), ctypes.byref(cfg)) == 2
    assert b"read failed" in lib.awq_last_error()
    # awq_create refuses the directory before any GPU call
    h = ctypes.c_void_p()
    assert lib.awq_create(d.encode(), ctypes.byref(cfg), ctypes.byref(h)) == 2 and not h.value
    # full-size totals of the reference layout
    full = awq.default_config()
    total = sum((n if (p == awq.P_PACKED and k != awq.T_GAMMA) else 2 * n)
                for (l, k, p) in awq.tensor_list(full) for n in [full.part_count(k, p)])
    assert total == 3642565388
    assert len(awq.tensor_list(full)) == 474


def test_bad_configs_are_rejected(awq, lib, tmp_path):
    for kw in [dict(hidden=500), dict(inter=100), dict(vocab=100), dict(max_pos=0), dict(n_layers=0),
               dict(max_pos=70000)]:
        base = dict(n_layers=2, hidden=512, inter=1024, vocab=1280, max_pos=16)
        base.update(kw)
        cfg = awq.make_config(**base)
        assert lib.awq_validate_weight_dir(str(tmp_path).encode(), ctypes.byref(cfg)) == 1, kw


def test_gemm_rejects_bad_arguments_before_any_gpu_call(lib):
    """awq_gemm's host checks (shape, alignment) fail with AWQ_ERR_ARG and a message; nothing is launched"""
    buf = ctypes.create_string_buffer(4096 + 64)
    base = (ctypes.addressof(buf) + 63) & ~63
    call = lambda wq, x, m, k, M: lib.awq_gemm(ctypes.c_void_p(wq), ctypes.c_void_p(base), ctypes.c_void_p(base), m, k,
                                              ctypes.c_void_p(x), ctypes.c_void_p(base), M, 1, None, None)
    assert call(base, base + 2, 4096, 4096, 40) == 1 and b"16-byte aligned" in lib.awq_last_error()
    assert call(base + 8, base, 12288, 4096, 40) == 1 and b"16-byte aligned" in lib.awq_last_error()
    assert call(base, base, 4096, 4000, 40) == 1 and b"multiples of 128" in lib.awq_last_error()
    assert call(base, base, 4096, 4096, 0) == 1 and b"M out of range" in lib.awq_last_error()
    assert call(base, base, 6144, 4096, 40) == 1 and b"scale group" in lib.awq_last_error()


def test_cli_usage_error():
    exe = os.path.join(ROOT, "cuda-kernel-qwen3-8b-awq_amd", "qwen3_awq_infer")
    res = subprocess.run([exe], capture_output=True, text=True)
    assert res.returncode == 1 and "Usage:" in res.stderr          # Inference.cu:1414-1417
    res = subprocess.run([exe, "/nonexistent-dir"], capture_output=True, text=True)
    assert res.returncode == 1 and "could not open" in res.stderr  # Inference.cu:299-302


def test_synth_matches_numpy_and_fixture(awq, lib):
    seed = 42
    fx = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "synth_seed42.json")))
    # packed bytes
    buf = np.zeros(1000, dtype=np.uint8)
    awq.check(lib.awq_synth_fill(seed, 3, awq.T_W1, awq.P_PACKED, ptr(buf), buf.size))
    assert np.array_equal(buf, helpers.synth_packed(seed, 3, awq.T_W1, 1000))
    assert buf[:16].tolist() == fx["w1_layer3_packed_first16"]
    # scale and zero-point
    sc = np.zeros(96, dtype=np.float16)
    awq.check(lib.awq_synth_fill(seed, 3, awq.T_W1, awq.P_SCALE, ptr(sc), sc.size))
    assert np.array_equal(sc.view(np.uint16), helpers.synth_scale(seed, 3, awq.T_W1, 96).view(np.uint16))
    assert sc[:8].view(np.uint16).tolist() == fx["w1_layer3_scale_first8_bits"]
    assert sc.min() >= 0.002 - 1e-5 and sc.max() <= 0.02
    zp = np.zeros(96, dtype=np.float16)
    awq.check(lib.awq_synth_fill(seed, 3, awq.T_W1, awq.P_ZP, ptr(zp), zp.size))
    assert np.array_equal(zp.view(np.uint16), helpers.synth_zp(seed, 3, awq.T_W1, 96).view(np.uint16))
    assert zp[:8].astype(int).tolist() == fx["w1_layer3_zp_first8"]
    assert set(np.unique(zp).tolist()) <= set(float(i) for i in range(16))
    # the two global tensors ignore the layer argument
    a = np.zeros(64, dtype=np.uint8); b = np.zeros(64, dtype=np.uint8)
    awq.check(lib.awq_synth_fill(seed, 0, awq.T_UNEMBED, awq.P_PACKED, ptr(a), 64))
    awq.check(lib.awq_synth_fill(seed, 7, awq.T_UNEMBED, awq.P_PACKED, ptr(b), 64))
    assert np.array_equal(a, b)
    # normals: numpy statement of the same Box-Muller, then distribution checks
    x = np.zeros(200000, dtype=np.float16)
    awq.check(lib.awq_synth_normal_f16(seed, awq.SYNTH_STREAM_INPUT, ptr(x), x.size, 0.0, 1.0))
    ref = helpers.synth_normal(seed, awq.SYNTH_STREAM_INPUT, x.size).astype(np.float16)
    assert np.mean(x.view(np.uint16) == ref.view(np.uint16)) > 0.9999
    assert abs(float(x.astype(np.float64).mean())) < 0.01 and abs(float(x.astype(np.float64).std()) - 1.0) < 0.01
    assert x[:8].view(np.uint16).tolist() == fx["normal_first8_bits"]
    g = np.zeros(4096, dtype=np.float16)
    awq.check(lib.awq_synth_fill(seed, 0, awq.T_GAMMA, 0, ptr(g), g.size))
    assert abs(float(g.astype(np.float64).mean()) - 1.0) < 2e-3 and abs(float(g.astype(np.float64).std()) - 0.02) < 2e-3
    # token ids
    t = np.zeros(128, dtype=np.int32)
    awq.check(lib.awq_synth_tokens(seed, awq.SYNTH_STREAM_INPUT + 1, ptr(t), t.size, 151936))
    h = helpers.synth_hash(seed, awq.SYNTH_STREAM_INPUT + 1, np.arange(128, dtype=np.uint64))
    assert np.array_equal(t, (h % np.uint64(151936)).astype(np.int32))
    assert t[:8].tolist() == fx["tokens_first8"]


def test_rope_tables_host_match_oracle(awq, lib, oracle):
    mp = 4096
    a, b = np.zeros((mp, 64), np.float16), np.zeros((mp, 64), np.float16)
    c, d = np.zeros((mp, 64), np.float16), np.zeros((mp, 64), np.float16)
    awq.check(lib.awq_rope_tables_host(ptr(a), ptr(b), mp))
    oracle.awqo_rope_tables(ptr(c), ptr(d), mp)
    assert np.array_equal(a.view(np.uint16), c.view(np.uint16)) and np.array_equal(b.view(np.uint16), d.view(np.uint16))


def test_workspace_size_queries_need_no_gpu(lib):
    """host-side arithmetic only: sizes of the scratch areas the kernel-level entry points take"""
    assert lib.awq_gemv_workspace_bytes(4096, 4096) == 256
    # a product with few output tiles may cut k over workgroups: a 4096-byte header (status word,
    # hand-over counters) and room for 4 partial results, or for one 256 x 128 tile of FP32 sums
    # per compute unit
    assert lib.awq_gemm_workspace_bytes(4096, 12288, 128) == 4096 + 4 * 128 * 4096 * 4
    assert lib.awq_gemm_workspace_bytes(4096, 12288, 1024) == 4096 + 256 * 256 * 128 * 4
    assert lib.awq_gemm_workspace_bytes(12288, 4096, 2048) == 0     # plenty of tiles: never cut
    assert lib.awq_gemm_workspace_bytes(4096, 4096, 4) == 0         # the few-token kernel
    heads, max_pos = 32, 40960
    chunks = (max_pos + 63) // 64
    assert lib.awq_attention_workspace_bytes(heads, max_pos) == heads * (max_pos + chunks * 129 + 32) * 4
    assert lib.awq_argmax_workspace_bytes(151936) > 0


def test_bench_refuses_more_than_one_gpu():
    """the benchmark measures one GPU; asking for more ends with a message, before anything touches a device"""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_gemm_plan_for_the_model_matrices(lib):
    """the workgroup shape awq_gemm picks (host arithmetic): the measured rules, on the model's matrices"""
    K_SPLIT, ROWS, ROWS_64, ROWS_CUT = 1, 2, 3, 4
    w1, w2, wo = (12288, 4096), (4096, 12288), (4096, 4096)
    plan = lambda shape, M, ws=1: lib.awq_gemm_plan(shape[0], shape[1], M, ws)
    assert plan(w1, 1) == 0 and plan((256, 512), 4) == 0 and plan((256, 512), 5) == K_SPLIT
    assert [plan(s, M) for s in (w1, w2, wo) for M in (2, 4, 16)] == [5] * 9   # k a multiple of 4096
    assert [plan(w1, M) for M in (17, 32, 33, 64, 65, 128, 200, 256)] == [7] * 8   # 64-row workgroups, tokens shared through LDS
    assert plan((12288, 2048), 50) == 7 and plan((12288, 8192), 50) == K_SPLIT and plan((8192, 4096), 50) == K_SPLIT
    assert [plan(w1, M) for M in (257, 384)] == [ROWS_64] * 2           # 96..144 tiles: units would idle
    assert [plan(w1, M) for M in (512, 640)] == [ROWS] * 2              # 192..240 tiles, one per unit
    assert [plan(w1, M) for M in (704, 1024)] == [ROWS_64] * 2          # 288..384 tiles: three per unit in one round
    assert [plan(w1, M) for M in (1280, 2048, 4096)] == [ROWS] * 3
    assert [plan(w2, M) for M in (64, 127, 512)] == [K_SPLIT] * 3
    assert [plan(w2, M) for M in (128, 192, 320)] == [8] * 3 and plan(w2, 192, 0) != 8   # k cut, sums in the workspace
    assert lib.awq_gemm_workspace_bytes(4096, 12288, 192) == 4096 + 4 * 192 * 4096 * 4
    assert [plan(w2, M) for M in (640, 1024, 1280)] == [ROWS_CUT] * 3   # long k, 80..160 tiles
    assert plan(w2, 1024, 0) == ROWS                                    # no workspace: no hand-over
    assert [plan(w2, M) for M in (2048, 4096)] == [ROWS] * 2
    assert [plan(wo, M) for M in (17, 32, 33, 64)] == [6] * 4           # tokens shared through LDS
    assert plan((4096, 2048), 40) == 6 and plan((4096, 8192), 40) == K_SPLIT and plan((8192, 4096), 40) == K_SPLIT
    assert lib.awq_gemm_workspace_bytes(4096, 4096, 40) == 0
    assert [plan(wo, M) for M in (65, 128, 193, 512)] == [K_SPLIT] * 4 and [plan(wo, M) for M in (129, 192)] == [6] * 2
    assert [plan(wo, M) for M in (576, 1024, 1280)] == [ROWS_64] * 3
    assert plan(wo, 2048) == ROWS and plan(wo, 2560) == ROWS_64 and plan(wo, 4096) == ROWS
