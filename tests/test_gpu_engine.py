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
