"""GPU parity of the whole engine against the CPU oracle: identical greedy token ids, identical
hidden state and logits (bit for bit), through the drop-in surface QWen3AWQInfer /
generateResponse and the weight directory of the reference."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

from helpers import fill_pair, make_oracle_model, ptr

pytestmark = pytest.mark.gpu


def oracle_generate(oracle, model, prompt, n_new):
    p = np.asarray(prompt, dtype=np.int32)
    out = np.zeros(max(1, n_new), dtype=np.int32)
    rc = oracle.awqo_model_generate(model, ptr(p) if p.size else None, p.size, n_new, ptr(out))
    assert rc == n_new
    return out[:n_new].tolist()


def compare_state(awq, oracle, eng, model, cfg):
    hid = np.ctypeslib.as_array(eng.read_hidden())
    oh = np.ctypeslib.as_array(ctypes.cast(oracle.awqo_model_last_layer_out(model), ctypes.POINTER(ctypes.c_uint16)), (cfg.hidden,))
    assert np.array_equal(hid, oh)
    lg = np.ctypeslib.as_array(eng.read_logits())
    ol = np.ctypeslib.as_array(ctypes.cast(oracle.awqo_model_logits(model), ctypes.POINTER(ctypes.c_uint16)), (cfg.vocab,))
    assert np.array_equal(lg, ol)


SMALL = dict(n_layers=4, hidden=512, inter=1536, vocab=1024, max_pos=128)


def test_small_model_sequence_crossing_the_attention_switch(awq, oracle, torch_gpu):
    """a 690-token prompt and 24 new tokens: the attended length passes 128 and 704, where the engine
    changes attention launches (and captured graph); tokens and state stay the oracle's.  Then a second,
    shorter sequence on the same engine, whose cache still holds the first one's rows past its own length."""
    cfg = awq.make_config(n_layers=2, hidden=512, inter=512, vocab=1024, max_pos=768)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 99, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    rng = np.random.default_rng(3)
    prompt = rng.integers(0, cfg.vocab, 690).tolist()
    print("small model, sequence crossing 704 positions", flush=True)
    got = eng.generateResponse(prompt, 24)
    ref = oracle_generate(oracle, model, prompt, 24)
    assert got == ref
    compare_state(awq, oracle, eng, model, cfg)
    prompt = rng.integers(0, cfg.vocab, 126).tolist()
    print("second sequence, 126 + 12 positions over the stale cache", flush=True)
    got = eng.generateResponse(prompt, 12)
    ref = oracle_generate(oracle, model, prompt, 12)
    assert got == ref
    compare_state(awq, oracle, eng, model, cfg)
    eng.close()
    oracle.awqo_model_destroy(model)


def test_results_do_not_depend_on_the_cache_capacity(awq, torch_gpu):
    """the engine keeps its key/value rows in blocks of 64 positions per head; whatever capacity the
    cache is allocated for (not a multiple of 64, the reference's 40,960), a sequence that crosses a
    block boundary gives the same tokens, hidden state and logits, prompt token by token or batched"""
    results = []
    for max_pos in (150, 1024, 40960):
        cfg = awq.make_config(n_layers=2, hidden=512, inter=512, vocab=1024, max_pos=max_pos)
        eng = awq.QWen3AWQInfer.empty(cfg)
        lib = awq.load_library()
        for layer, kind, part in awq.tensor_list(cfg):
            count = cfg.part_count(kind, part)
            nbytes = count if (part == awq.P_PACKED and kind != awq.T_GAMMA) else 2 * count
            buf = (ctypes.c_uint8 * nbytes)()
            awq.check(lib.awq_synth_fill_profile(awq.SYNTH_BALANCED, 7, layer, kind, part, buf, count))
            eng.upload(layer, kind, part, buf, nbytes)
        eng.finalize()
        rng = np.random.default_rng(11)
        prompt = rng.integers(0, cfg.vocab, 100).tolist()
        for batched in (False, True):
            eng.set_prefill_mode(batched)
            print("cache capacity", max_pos, "batched prompt", batched, flush=True)
            toks = eng.generateResponse(prompt, 40)
            results.append((max_pos, batched, toks, np.ctypeslib.as_array(eng.read_hidden()).copy(),
                            np.ctypeslib.as_array(eng.read_logits()).copy()))
        eng.close()
    for batched in (False, True):
        same = [r for r in results if r[1] == batched]
        for r in same[1:]:
            assert r[2] == same[0][2]
            assert np.array_equal(r[3], same[0][3]) and np.array_equal(r[4], same[0][4])


@pytest.mark.parametrize("graph", [False, True])
def test_small_model_tokens_and_state_identical(awq, oracle, torch_gpu, graph):
    cfg = awq.make_config(**SMALL)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 1234, engine=eng, model=model)
    eng.set_graph_mode(graph)
    prompt = [3, 1000, 77, 512, 9]
    print("small model generate graph=", graph, flush=True)
    got = eng.generateResponse(prompt, 24)
    ref = oracle_generate(oracle, model, prompt, 24)
    assert got == ref
    compare_state(awq, oracle, eng, model, cfg)
    # a second call starts from a clean sequence and gives the same answer
    assert eng.generateResponse(prompt, 24) == ref
    # edge cases: empty prompt, single token prompt, zero new tokens
    assert eng.generateResponse([], 5) == oracle_generate(oracle, model, [], 5)
    assert eng.generateResponse([1], 3) == oracle_generate(oracle, model, [1], 3)
    assert eng.generateResponse([1, 2], 0) == []
    with pytest.raises(awq.AwqError):
        eng.generateResponse([1] * 100, 29)   # 129 > max_pos
    with pytest.raises(awq.AwqError):
        eng.generateResponse([5000], 1)       # id outside the vocabulary
    eng.close()
    oracle.awqo_model_destroy(model)


@pytest.mark.parametrize("graph", [False, True])
def test_decode_in_pieces_equals_one_call(awq, oracle, torch_gpu, graph):
    """awq_decode leaves the next step's state and input on the device (the sampled token's embedding in the
    hidden buffer, the advanced position and lengths), and the host writes the state once per call: a
    generation cut into calls of 1, 2, 0, 5 and 16 steps, with the hidden state and the logits read in
    between, gives the tokens and the state of one call.  Also without a prompt, where the first step
    starts from the zero hidden state."""
    cfg = awq.make_config(**SMALL)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 4321, engine=eng, model=model)
    eng.set_graph_mode(graph)
    for prompt in ([3, 1000, 77, 512, 9], []):
        pieces = (1, 2, 0, 5, 16)
        print("piecewise decode graph=", graph, "prompt", prompt, flush=True)
        eng.reset()
        eng.prefill(prompt)
        got = []
        for n in pieces:
            got += eng.decode(n)
            ref = oracle_generate(oracle, model, prompt, len(got))
            assert got == ref
            if got:
                compare_state(awq, oracle, eng, model, cfg)   # reading does not disturb the sequence
        assert len(set(got)) > 1
    with pytest.raises(awq.AwqError):
        eng.prefill([1])            # prompt tokens cannot follow generated ones
    eng.close()
    oracle.awqo_model_destroy(model)


def test_unembed_period_model(awq, oracle, torch_gpu):
    """vocab/128 coprime to hidden/128 gives the unembedding the j-dependent scale groups of the
    real 151936 x 4096 matrix"""
    cfg = awq.make_config(n_layers=2, hidden=512, inter=512, vocab=128 * 37, max_pos=64)
    assert oracle.awqo_group_period(cfg.vocab, cfg.hidden) == 4
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 99, engine=eng, model=model)
    prompt = [4000, 17, 300]
    assert eng.generateResponse(prompt, 16) == oracle_generate(oracle, model, prompt, 16)
    compare_state(awq, oracle, eng, model, cfg)
    eng.close()
    oracle.awqo_model_destroy(model)


def test_weight_directory_round_trip_and_cli(awq, lib, oracle, torch_gpu, tmp_path):
    """the drop-in path: files named and sized as Inference.cu:780-899, loaded by awq_create and by
    the command-line harness; a short file is an error before any GPU work"""
    cfg = awq.make_config(**SMALL)
    d = str(tmp_path / "weights")
    os.makedirs(d)
    awq.check(lib.awq_write_weight_dir(d.encode(), ctypes.byref(cfg), 777))
    assert os.path.getsize(os.path.join(d, "layer_0_wqkv.bin")) == 3 * 512 * 512 // 2
    assert os.path.getsize(os.path.join(d, "layer_3_bqkv_scale.bin")) == (3 * 512 // 128) * 2
    assert os.path.getsize(os.path.join(d, "rms_norm_gamma_2.bin")) == 1024
    assert os.path.getsize(os.path.join(d, "unembed_zp.bin")) == (1024 // 128) * 2
    eng = awq.QWen3AWQInfer(d, config=cfg)
    model = make_oracle_model(oracle, cfg)
    assert oracle.awqo_model_load_dir(model, d.encode()) == 0
    prompt = [1, 2, 3]
    assert eng.generateResponse(prompt, 12) == oracle_generate(oracle, model, prompt, 12)
    eng.close()
    # the engine built from in-memory synthetic weights of the same seed is the same model
    eng2 = awq.QWen3AWQInfer.from_synthetic(cfg, 777)
    assert eng2.generateResponse(prompt, 12) == oracle_generate(oracle, model, prompt, 12)
    eng2.close()
    oracle.awqo_model_destroy(model)
    # truncated file -> error, nothing loaded
    with open(os.path.join(d, "layer_1_w2.bin"), "r+b") as f:
        f.truncate(100)
    with pytest.raises(awq.AwqError) as ei:
        awq.QWen3AWQInfer(d, config=cfg)
    assert ei.value.code == 2 and "layer_1_w2.bin" in str(ei.value)


def test_drop_in_class_and_command_line_on_the_full_size_directory(awq, lib, oracle, torch_gpu, tmp_path):
    """The reference's own use (Inference.cu:1413-1433): main() builds QWen3AWQInfer(argv[1]) on a directory
    in the README layout (474 headerless files, 3,642,565,388 bytes), calls generateResponse({151643}, 20) and
    prints "Generated tokens: " followed by the ids.  Here the built command-line harness runs as a child
    process on such a directory and its 20 ids must be the CPU oracle's on the same files; the engine that
    awq_create loads from the directory (pinned double-buffered loader) must then be in the same state, bit
    for bit, as one filled through awq_upload from memory."""
    cfg = awq.default_config()
    d = str(tmp_path / "qwen3_awq_weights")
    os.makedirs(d)
    seed = 2025
    print("writing the 3.64 GB weight directory", flush=True)
    awq.check(lib.awq_write_weight_dir_profile(d.encode(), ctypes.byref(cfg), seed, awq.SYNTH_BALANCED))
    total = sum(os.path.getsize(os.path.join(d, f)) for f in os.listdir(d))
    assert len(os.listdir(d)) == 474 and total == 3642565388          # README sizes, Inference.cu:780-899
    cli = os.path.join(os.path.dirname(awq.LIB_PATH), "qwen3_awq_infer")
    print("running", cli, flush=True)
    res = subprocess.run([cli, d], capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, res.stderr
    line = [ln for ln in res.stdout.splitlines() if ln.startswith("Generated tokens: ")]
    assert len(line) == 1 and res.stdout.endswith(" \n")               # ids separated and followed by a space
    got = [int(t) for t in line[0][len("Generated tokens: "):].split()]
    # the oracle on the same files (its cache only needs the 21 positions of this run)
    ocfg = awq.make_config(max_pos=32)
    model = make_oracle_model(oracle, ocfg)
    assert oracle.awqo_model_load_dir(model, d.encode()) == 0
    ref = oracle_generate(oracle, model, [151643], 20)
    print("command line:", got, flush=True)
    assert got == ref
    assert len(set(got)) > 1                                             # not a collapsed sequence
    # awq_create(dir) against awq_upload of the same bytes: ids, hidden state and logits
    eng = awq.QWen3AWQInfer(d, config=ocfg)
    assert 0.0 < lib.awq_last_load_seconds() < 120.0
    print("directory loaded in %.2f s" % lib.awq_last_load_seconds(), flush=True)
    a = eng.generateResponse([151643, 7, 99], 8)
    ha, la = np.ctypeslib.as_array(eng.read_hidden()).copy(), np.ctypeslib.as_array(eng.read_logits()).copy()
    eng.close()
    eng2 = awq.QWen3AWQInfer.empty(ocfg)
    fill_pair(awq, oracle, ocfg, seed, engine=eng2, model=model, profile=awq.SYNTH_BALANCED)
    b = eng2.generateResponse([151643, 7, 99], 8)
    hb, lb = np.ctypeslib.as_array(eng2.read_hidden()).copy(), np.ctypeslib.as_array(eng2.read_logits()).copy()
    eng2.close()
    assert a == b and np.array_equal(ha, hb) and np.array_equal(la, lb)
    assert a == oracle_generate(oracle, model, [151643, 7, 99], 8)
    oracle.awqo_model_destroy(model)
    # a file that is too short stops the loader with the reference's message, before anything runs
    with open(os.path.join(d, "layer_35_w2_zp.bin"), "r+b") as f:
        f.truncate(10)
    res = subprocess.run([cli, d], capture_output=True, text=True, timeout=600)
    assert res.returncode == 1 and "layer_35_w2_zp.bin" in res.stderr


@pytest.mark.parametrize("n_layers,prompt_len,n_new", [(2, 3, 6)])
def test_full_width_model_token_identity(awq, oracle, torch_gpu, n_layers, prompt_len, n_new):
    """reference widths (hidden 4096, intermediate 12288, vocabulary 151936), fewer layers"""
    cfg = awq.make_config(n_layers=n_layers, max_pos=64)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 2024, engine=eng, model=model)
    prompt = np.zeros(prompt_len, dtype=np.int32)
    awq.check(awq.load_library().awq_synth_tokens(2024, awq.SYNTH_STREAM_INPUT, ptr(prompt), prompt_len, cfg.vocab))
    print("full width generate", flush=True)
    got = eng.generateResponse(prompt.tolist(), n_new)
    ref = oracle_generate(oracle, model, prompt.tolist(), n_new)
    assert got == ref
    compare_state(awq, oracle, eng, model, cfg)
    eng.close()
    oracle.awqo_model_destroy(model)


def test_config2_one_decoder_layer_at_position_512(awq, lib, oracle, torch_gpu):
    """config 2: one full decoder layer at decode batch 1, reference widths, 512 prior cached positions of
    N(0,1) values, attention over L = 513 -- composed from the C ABI's kernel entry points exactly as
    runOneLayer (Inference.cu:1029-1230) orders them, against the oracle's layer"""
    import ctypes as C
    torch = torch_gpu
    H, I, nh, mp, pos, L = 4096, 12288, 32, 640, 512, 513
    cfg = awq.make_config(n_layers=1, max_pos=mp, vocab=128)
    model = make_oracle_model(oracle, cfg)
    fill_pair(awq, oracle, cfg, 4242, engine=None, model=model)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def host(kind, part):
        n = C.c_int64(0)
        p = oracle.awqo_model_tensor(model, 0, kind, part, C.byref(n))
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), (n.value,))

    def upload(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    # seeded inputs: hidden state and the first 512 cache rows of every head
    hidden = np.zeros(H, dtype=np.float16)
    awq.check(lib.awq_synth_normal_f16(4242, awq.SYNTH_STREAM_INPUT + 2, ptr(hidden), H, 0.0, 1.0))
    kv = np.zeros((2, nh, mp, 128), dtype=np.float16)
    for which in range(2):
        rows = np.zeros((nh, pos, 128), dtype=np.float16)
        awq.check(lib.awq_synth_normal_f16(4242, awq.SYNTH_STREAM_INPUT + 3 + which, ptr(rows), rows.size, 0.0, 1.0))
        kv[which, :, :pos] = rows
    for which, getter in ((0, oracle.awqo_model_kcache), (1, oracle.awqo_model_vcache)):
        dst = np.ctypeslib.as_array(C.cast(getter(model, 0), C.POINTER(C.c_uint16)), (nh * mp * 128,))
        dst[:] = kv[which].reshape(-1).view(np.uint16)
    oh = np.ctypeslib.as_array(C.cast(oracle.awqo_model_hidden_mut(model), C.POINTER(C.c_uint16)), (H,))
    oh[:] = hidden.view(np.uint16)
    oracle.awqo_model_layer(model, 0, pos, L)
    ref_hidden = oh.copy()
    ref_k = np.ctypeslib.as_array(C.cast(oracle.awqo_model_kcache(model, 0), C.POINTER(C.c_uint16)), (nh * mp * 128,)).copy()

    # device side
    dims = {awq.T_WQKV: (3 * H, H), awq.T_WO: (H, H), awq.T_W1: (I, H), awq.T_W2: (H, I)}
    dev_w = {}
    for kind, (m, k) in dims.items():
        d_in = upload(host(kind, awq.P_PACKED))
        d_w = torch.empty_like(d_in)
        awq.check(lib.awq_linear_repack(d_in.data_ptr(), d_w.data_ptr(), m, k, st))
        dev_w[kind] = (d_w, upload(host(kind, awq.P_SCALE)), upload(host(kind, awq.P_ZP)))
    d_gamma = upload(host(awq.T_GAMMA, 0))
    cos_t, sin_t = np.zeros((mp, 64), np.float16), np.zeros((mp, 64), np.float16)
    awq.check(lib.awq_rope_tables_host(ptr(cos_t), ptr(sin_t), mp))
    d_cos, d_sin = upload(cos_t), upload(sin_t)
    d_k, d_v = upload(kv[0]), upload(kv[1])
    d_hidden = upload(hidden)
    d_q = torch.zeros(H, dtype=torch.float16, device="cuda")
    d_ctx = torch.zeros(H, dtype=torch.float16, device="cuda")
    d_mid = torch.zeros(I, dtype=torch.float16, device="cuda")
    ws = torch.zeros(lib.awq_gemv_workspace_bytes(H, H), dtype=torch.uint8, device="cuda")
    att_ws = torch.zeros(lib.awq_attention_workspace_bytes(nh, mp), dtype=torch.uint8, device="cuda")

    def linear(kind, x, y, **kw):
        a = awq.AwqLinearArgs()
        w, s, z = dev_w[kind]
        a.repacked, a.scale, a.zp = w.data_ptr(), s.data_ptr(), z.data_ptr()
        a.m, a.k = dims[kind]
        a.x, a.y, a.workspace, a.eps = x.data_ptr(), y.data_ptr(), ws.data_ptr(), 1e-6
        for key, val in kw.items():
            setattr(a, key, val)
        awq.check(lib.awq_gemv_fused(C.byref(a), st))

    linear(awq.T_WQKV, d_hidden, d_q, prologue=awq.PRO_RMSNORM, gamma=d_gamma.data_ptr(), epilogue=awq.EPI_QKV_ROPE,
           cos_t=d_cos.data_ptr(), sin_t=d_sin.data_ptr(), k_cache=d_k.data_ptr(), v_cache=d_v.data_ptr(),
           hidden=H, max_pos=mp, pos=pos)
    awq.check(lib.awq_decode_attention(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), d_ctx.data_ptr(), nh, mp, L,
                                       att_ws.data_ptr(), st))
    linear(awq.T_WO, d_ctx, d_hidden, epilogue=awq.EPI_RESIDUAL, residual=d_hidden.data_ptr())
    linear(awq.T_W1, d_hidden, d_mid, prologue=awq.PRO_RMSNORM, gamma=d_gamma.data_ptr(), epilogue=awq.EPI_GELU)
    linear(awq.T_W2, d_mid, d_hidden, epilogue=awq.EPI_RESIDUAL, residual=d_hidden.data_ptr())
    torch.cuda.synchronize()
    assert np.array_equal(d_hidden.cpu().numpy().view(np.uint16), ref_hidden)
    assert np.array_equal(d_k.cpu().numpy().reshape(-1).view(np.uint16), ref_k)
    oracle.awqo_model_destroy(model)


def test_full_model_32_greedy_tokens_identical(awq, oracle, torch_gpu):
    """config 4 at reduced length: all 36 layers at the reference widths, random-init seeded weights, greedy
    decode of 32 tokens; ids, final hidden state and last logits must equal the CPU path bit for bit.
    Weights come from the balanced profile (include/awq_synth.h): with the benchmark's own distributions the
    activations overflow binary16 by layer 3 and every token is 0, which would test nothing (that regime is
    covered by the next test).  Here the logits are finite and the top-1/top-2 margin is a few FP16 ulps, so
    any rounding difference between the two paths changes the ids."""
    cfg = awq.make_config(max_pos=64)
    assert (cfg.n_layers, cfg.hidden, cfg.inter, cfg.vocab, cfg.split_idx) == (36, 4096, 12288, 151936, 18)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 2025, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    prompt = np.zeros(4, dtype=np.int32)
    awq.check(awq.load_library().awq_synth_tokens(2025, awq.SYNTH_STREAM_INPUT, ptr(prompt), prompt.size, cfg.vocab))
    print("36-layer model: 32 greedy tokens", flush=True)
    got = eng.generateResponse(prompt.tolist(), 32)
    ref = oracle_generate(oracle, model, prompt.tolist(), 32)
    margins = np.zeros(64, dtype=np.float32)
    n = oracle.awqo_model_margins(model, ptr(margins), 64)
    print("top-1/top-2 logit margins: min %.4f median %.4f" % (margins[:n].min(), np.median(margins[:n])), flush=True)
    assert got == ref
    assert len(set(got)) > 1 and np.isfinite(margins[:n]).all() and margins[:n].min() < 0.5
    compare_state(awq, oracle, eng, model, cfg)
    eng.close()
    oracle.awqo_model_destroy(model)


def test_config4_at_its_stated_length(awq, oracle, torch_gpu):
    """config 4 as the benchmark definition states it: all 36 layers at the reference widths, a prompt of
    128 token ids uniform in [0, 151936), 256 new tokens greedily at batch 1 -- 384 forward passes of
    generateResponse (Inference.cu:1297-1408) on both paths; all 256 ids, the last layer's output and the
    last logits must be the CPU path's bit for bit"""
    cfg = awq.make_config(max_pos=384)
    assert (cfg.n_layers, cfg.hidden, cfg.inter, cfg.vocab, cfg.split_idx) == (36, 4096, 12288, 151936, 18)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 31, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    prompt = np.zeros(128, dtype=np.int32)
    awq.check(awq.load_library().awq_synth_tokens(31, awq.SYNTH_STREAM_INPUT, ptr(prompt), prompt.size, cfg.vocab))
    assert prompt.min() >= 0 and prompt.max() < cfg.vocab and len(set(prompt.tolist())) > 100
    print("36-layer model: 128-token prompt, 256 greedy tokens on the GPU", flush=True)
    got = eng.generateResponse(prompt.tolist(), 256)
    print("the same on the CPU oracle (384 forward passes)", flush=True)
    ref = oracle_generate(oracle, model, prompt.tolist(), 256)
    margins = np.zeros(256, dtype=np.float32)
    n = oracle.awqo_model_margins(model, ptr(margins), 256)
    print("distinct ids %d, top-1/top-2 logit margins: min %.4f median %.4f" %
          (len(set(ref)), margins[:n].min(), np.median(margins[:n])), flush=True)
    assert len(got) == 256 and got == ref
    assert len(set(got)) > 1 and np.isfinite(margins[:n]).all()
    compare_state(awq, oracle, eng, model, cfg)
    eng.close()
    oracle.awqo_model_destroy(model)


def test_full_model_benchmark_distributions_overflow_identically(awq, oracle, torch_gpu):
    """the benchmark's own value distributions on the 36-layer model: activations reach inf/NaN within four
    layers on both paths; the hidden state, the logits (NaN patterns included) and the ids still agree"""
    cfg = awq.make_config(max_pos=32)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 2026, engine=eng, model=model, profile=awq.SYNTH_SPEC)
    prompt = [151643, 17]
    got = eng.generateResponse(prompt, 6)
    assert got == oracle_generate(oracle, model, prompt, 6)
    compare_state(awq, oracle, eng, model, cfg)
    eng.close()
    oracle.awqo_model_destroy(model)


def test_non_integral_zero_points_take_the_general_dequantisation(awq, oracle, torch_gpu):
    """AWQ zero-points are integers, which the kernels exploit (two exact operations instead of
    three); a checkpoint with fractional zero-points must be detected at upload and still give the
    oracle's bits through the general sequence"""
    cfg = awq.make_config(**SMALL)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)

    def fractional(layer, kind, part, address, count):
        if part == awq.P_ZP and kind != awq.T_GAMMA:
            z = np.ctypeslib.as_array(ctypes.cast(address, ctypes.POINTER(ctypes.c_uint16)), (count,)).view(np.float16)
            z += np.float16(0.25) * ((np.arange(count) % 3) + 1).astype(np.float16)

    fill_pair(awq, oracle, cfg, 4321, engine=eng, model=model, profile=awq.SYNTH_BALANCED, mutate=fractional)
    prompt = [9, 100, 1000]
    print("fractional zero-points", flush=True)
    got = eng.generateResponse(prompt, 12)
    assert got == oracle_generate(oracle, model, prompt, 12)
    compare_state(awq, oracle, eng, model, cfg)
    eng.close()
    oracle.awqo_model_destroy(model)


def test_fused_wo_w1_launch_is_bit_identical_and_gives_up_cleanly(awq, lib, oracle, torch_gpu):
    """awq_set_fused_mode(e, 1): Wo + residual and RMSNorm + W1 + GeLU of a layer as one launch whose 256
    workgroups hand the hidden state to each other through memory (tagged words, bounded waits).  Two
    full-width layers: ids, hidden state and logits must be the oracle's bit for bit, with and without a
    captured graph, over enough steps for the tags to change a few hundred times.  Then the give-up path,
    driven from the host (the status word is set before the call, so every wait ends at its first look and
    every kernel runs to its end): the call fails with AWQ_ERR_HIP and the engine works again after a reset.
    Last, the instrumented launch behind awq_debug_fused_timeline returns ordered time stamps."""
    cfg = awq.make_config(n_layers=2, max_pos=256)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 2025, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    assert not eng.fused_mode() & eng.FUSED_WO_W1    # Wo and W1 are two launches by default
    eng.set_fused_mode(eng.FUSED_WO_W1)
    if not eng.fused_mode() & eng.FUSED_WO_W1:
        pytest.skip("this device cannot hold the fused launch's 256 workgroups at once")
    rng = np.random.default_rng(17)
    prompt = rng.integers(0, cfg.vocab, 40).tolist()
    for graph in (True, False):
        eng.set_graph_mode(graph)
        print("fused launch, graph", graph, flush=True)
        got = eng.generateResponse(prompt, 100)
        ref = oracle_generate(oracle, model, prompt, 100)
        print("distinct ids:", len(set(got)), flush=True)
        assert got == ref
        compare_state(awq, oracle, eng, model, cfg)
    eng.set_graph_mode(True)
    print("fused launch, every wait giving up", flush=True)
    eng.reset()
    awq.check(lib.awq_debug_force_handover_giveup(eng._h, 1))
    with pytest.raises(awq.AwqError) as ei:
        eng.prefill(prompt[:3])
    assert ei.value.code == 3 and "gave up" in str(ei.value)
    print("fused launch, after a reset", flush=True)
    assert eng.generateResponse(prompt, 100) == ref
    compare_state(awq, oracle, eng, model, cfg)
    # the same model through two launches per layer pair: the same bits
    eng.set_fused_mode(False)
    assert eng.generateResponse(prompt, 100) == ref
    buf = np.zeros(256 * 16, dtype=np.uint64)
    nw, ns = ctypes.c_int32(0), ctypes.c_int32(0)
    awq.check(lib.awq_debug_fused_timeline(eng._h, 1, buf.ctypes.data_as(ctypes.c_void_p), ctypes.byref(nw),
                                           ctypes.byref(ns)))
    t = buf[:nw.value * ns.value].reshape(nw.value, ns.value).astype(np.int64)
    assert nw.value == 256 and ns.value >= 8 and (np.diff(t, axis=1) >= 0).all()
    assert 0 < (t[:, -1].max() - t[:, 0].min()) * 0.01 < 1000.0     # microseconds
    eng.close()
    oracle.awqo_model_destroy(model)


def test_fused_qkv_attention_launch_is_bit_identical_and_gives_up_cleanly(awq, lib, oracle, torch_gpu):
    """awq_set_fused_mode(e, 2): RMSNorm + Wqkv + rotary + KV append and the attention of a layer as one launch
    (eight workgroups per head on one die, partial scores handed over through its L2, bounded waits).  Two
    full-width layers, a 40-token prompt token by token and 100 generated tokens (attended lengths on both sides
    of 128): ids, hidden state and logits must be the oracle's bit for bit, with and without a captured graph,
    also together with the fused Wo + W1 launch.  Then the give-up path, driven from the host (the status word
    is set before the call, so every wait ends at its first look and every kernel runs to its end): the call
    fails with AWQ_ERR_HIP and the engine works again after a reset.  Last, the instrumented launch behind
    awq_debug_qkv_attention_timeline returns ordered time stamps."""
    cfg = awq.make_config(n_layers=2, max_pos=1152)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 2025, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    if not eng.fused_mode() & eng.FUSED_QKV_ATTN:    # the default where the device can run it
        pytest.skip("this device cannot run the fused launch")
    eng.set_fused_mode(eng.FUSED_QKV_ATTN)
    rng = np.random.default_rng(17)
    prompt = rng.integers(0, cfg.vocab, 40).tolist()
    ref = oracle_generate(oracle, model, prompt, 100)
    for graph in (True, False):
        eng.set_graph_mode(graph)
        print("fused Wqkv + attention launch, graph", graph, flush=True)
        assert eng.generateResponse(prompt, 100) == ref
        compare_state(awq, oracle, eng, model, cfg)
    eng.set_graph_mode(True)
    eng.set_fused_mode(eng.FUSED_QKV_ATTN | eng.FUSED_WO_W1)
    if eng.fused_mode() == 3:
        print("both fused launches", flush=True)
        assert eng.generateResponse(prompt, 100) == ref
        compare_state(awq, oracle, eng, model, cfg)
    eng.set_fused_mode(eng.FUSED_QKV_ATTN)
    print("fused Wqkv + attention launch, every wait giving up", flush=True)
    eng.reset()
    awq.check(lib.awq_debug_force_handover_giveup(eng._h, 1))
    with pytest.raises(awq.AwqError) as ei:
        eng.prefill(prompt[:3])
    assert ei.value.code == 3 and "gave up" in str(ei.value)
    print("fused Wqkv + attention launch, after a reset", flush=True)
    assert eng.generateResponse(prompt, 100) == ref
    compare_state(awq, oracle, eng, model, cfg)
    # the drop-in call does not fail where the reference would not: after a give-up it runs the request again
    # with every launch on its own and leaves the fused launches off
    print("generateResponse over a give-up", flush=True)
    awq.check(lib.awq_debug_force_handover_giveup(eng._h, 2))
    assert eng.generateResponse(prompt, 100) == ref
    compare_state(awq, oracle, eng, model, cfg)
    assert eng.fused_mode() == 0
    awq.check(lib.awq_debug_force_handover_giveup(eng._h, 0))
    eng.set_fused_mode(eng.FUSED_QKV_ATTN)
    assert eng.fused_mode() == eng.FUSED_QKV_ATTN
    assert eng.generateResponse(prompt, 100) == ref
    buf = np.zeros(256 * 16, dtype=np.uint64)
    nw, ns = ctypes.c_int32(0), ctypes.c_int32(0)
    awq.check(lib.awq_debug_qkv_attention_timeline(eng._h, 1, 200, buf.ctypes.data_as(ctypes.c_void_p),
                                                   ctypes.byref(nw), ctypes.byref(ns)))
    t = buf[:nw.value * ns.value].reshape(nw.value, ns.value).astype(np.int64)
    assert nw.value == 256 and ns.value >= 8 and (np.diff(t, axis=1) >= 0).all()
    assert 0 < (t[:, -1].max() - t[:, 0].min()) * 0.01 < 1000.0     # microseconds
    # a long prompt token by token: attended lengths up to 1060, across the 704 and the 1024 at which the separate
    # attention switches from one launch to two and to three (the fused launch covers all of them, with a second
    # chunk of 64 positions per wavefront beyond 1024)
    eng.set_fused_mode(eng.FUSED_QKV_ATTN)
    long_prompt = rng.integers(0, cfg.vocab, 1010).tolist()
    print("fused Wqkv + attention launch, 1010-token prompt", flush=True)
    assert eng.generateResponse(long_prompt, 50) == oracle_generate(oracle, model, long_prompt, 50)
    compare_state(awq, oracle, eng, model, cfg)
    eng.set_fused_mode(0)
    assert eng.generateResponse(prompt, 100) == ref
    eng.close()
    oracle.awqo_model_destroy(model)


def test_fused_qkv_attention_launch_over_the_wrap_of_its_tags(awq, lib, torch_gpu):
    """The partial scores travel as words that carry a 16-bit tag, 1 + (launch counter mod 65535): the 36-layer
    model uses 36 tags per step, so a sequence of 1900 generated tokens passes the wrap (and the length bounds at
    128, 704 and 1024 positions, four steps per graph launch).  Ids, last hidden state and logits are those of the
    same sequence with Wqkv and the attention as separate launches, bit for bit."""
    cfg = awq.make_config(n_layers=36, max_pos=2048)
    eng = awq.QWen3AWQInfer.empty(cfg)
    for layer, kind, part in awq.tensor_list(cfg):
        count = cfg.part_count(kind, part)
        nbytes = count if (part == awq.P_PACKED and kind != awq.T_GAMMA) else 2 * count
        buf = (ctypes.c_uint8 * nbytes)()
        awq.check(lib.awq_synth_fill_profile(awq.SYNTH_BALANCED, 31, layer, kind, part, buf, count))
        eng.upload(layer, kind, part, buf, nbytes)
    eng.finalize()
    if not eng.fused_mode() & eng.FUSED_QKV_ATTN:
        pytest.skip("this device cannot run the fused launch")
    prompt = [11, 7, 1999, 3, 150000, 42, 8, 77]
    out = []
    for mode in (eng.FUSED_QKV_ATTN, 0):
        print("1900 generated tokens, fused mode", mode, flush=True)
        eng.set_fused_mode(mode)
        eng.reset()
        eng.prefill(prompt, batched=True)
        ids = eng.decode(1900)
        out.append((list(ids), np.ctypeslib.as_array(eng.read_hidden()).copy(),
                    np.ctypeslib.as_array(eng.read_logits()).copy()))
    assert out[0][0] == out[1][0] and len(set(out[0][0])) > 1
    assert np.array_equal(out[0][1], out[1][1]) and np.array_equal(out[0][2], out[1][2])
    eng.close()


def test_fused_qkv_attention_launch_across_its_length_bounds(awq, lib, torch_gpu):
    """The fused Wqkv + attention launch against the two launches it replaces (those are checked against the oracle
    at these lengths elsewhere) on sequences that cross 2048 and 3072 positions (a third and a fourth chunk of 64
    positions per wavefront) and 4096 (where the engine goes back to two launches): a batched prompt pass fills the caches and
    the launch's second copy of them, then generation steps.  Ids, last hidden state and logits bit for bit."""
    cfg = awq.make_config(n_layers=2, max_pos=4224)
    eng = awq.QWen3AWQInfer.empty(cfg)
    for layer, kind, part in awq.tensor_list(cfg):
        count = cfg.part_count(kind, part)
        nbytes = count if (part == awq.P_PACKED and kind != awq.T_GAMMA) else 2 * count
        buf = (ctypes.c_uint8 * nbytes)()
        awq.check(lib.awq_synth_fill_profile(awq.SYNTH_BALANCED, 77, layer, kind, part, buf, count))
        eng.upload(layer, kind, part, buf, nbytes)
    eng.finalize()
    if not eng.fused_mode() & eng.FUSED_QKV_ATTN:
        pytest.skip("this device cannot run the fused launch")
    rng = np.random.default_rng(5)
    for n_prompt, n_new in ((2020, 60), (3040, 60), (4070, 60)):
        prompt = rng.integers(0, cfg.vocab, n_prompt).tolist()
        out = []
        for mode in (0, eng.FUSED_QKV_ATTN):
            print("prompt", n_prompt, "fused mode", mode, flush=True)
            eng.reset()
            eng.set_fused_mode(mode)
            eng.prefill(prompt, batched=True)
            ids = eng.decode(n_new)
            out.append((list(ids), np.ctypeslib.as_array(eng.read_hidden()).copy(),
                        np.ctypeslib.as_array(eng.read_logits()).copy()))
        assert out[0][0] == out[1][0] and len(set(out[0][0])) > 1
        assert np.array_equal(out[0][1], out[1][1]) and np.array_equal(out[0][2], out[1][2])
    # the mode switched on in the middle of a sequence: the rows the two launches appended are copied over
    eng.reset()
    eng.set_fused_mode(0)
    eng.prefill(prompt[:2500], batched=True)
    a = list(eng.decode(20))
    eng.set_fused_mode(eng.FUSED_QKV_ATTN)
    b = list(eng.decode(20))
    eng.reset()
    eng.set_fused_mode(0)
    eng.prefill(prompt[:2500], batched=True)
    assert list(eng.decode(40)) == a + b
    eng.close()
