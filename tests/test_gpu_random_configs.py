"""Differential test over random small model shapes: the engine's greedy ids, final hidden state and
logits must be the CPU oracle's bit for bit, whatever the widths, layer count, vocabulary (including
vocabularies whose unembedding scale group depends on the input index), prompt length and launch
mode; the batched prompt pass must stay within rounding noise of the sequential one."""
import ctypes

import numpy as np
import pytest

from helpers import fill_pair, make_oracle_model, ptr

pytestmark = pytest.mark.gpu


def _cases():
    rng = np.random.default_rng(20240607)
    out = []
    for i in range(12):
        hidden = int(rng.choice([512, 1024]))
        inter = hidden * int(rng.choice([1, 2, 3]))
        n_layers = int(rng.integers(1, 4))
        vocab = int(rng.choice([256, 1024, 128 * 37, 128 * 9])) if hidden == 512 else int(rng.choice([512, 2048]))
        n_prompt = int(rng.choice([0, 1, 2, 7, 33, 70]))
        n_new = int(rng.integers(3, 12))
        out.append((i, hidden, inter, n_layers, vocab, n_prompt, n_new, bool(i & 1)))
    return out


@pytest.mark.parametrize("case,hidden,inter,n_layers,vocab,n_prompt,n_new,graph", _cases())
def test_random_shape_matches_oracle(awq, oracle, torch_gpu, case, hidden, inter, n_layers, vocab, n_prompt, n_new,
                                     graph):
    cfg = awq.make_config(n_layers=n_layers, hidden=hidden, inter=inter, vocab=vocab, max_pos=96,
                          split_idx=max(1, n_layers // 2))
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 500 + case, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    eng.set_graph_mode(graph)
    rng = np.random.default_rng(case)
    prompt = rng.integers(0, vocab, n_prompt).astype(np.int32)
    print("random shape", case, hidden, inter, n_layers, vocab, n_prompt, n_new, graph, flush=True)
    got = eng.generateResponse(prompt.tolist(), n_new)
    ref = np.zeros(n_new, dtype=np.int32)
    assert oracle.awqo_model_generate(model, ptr(prompt) if n_prompt else None, n_prompt, n_new, ptr(ref)) == n_new
    assert got == ref.tolist()
    hid = np.ctypeslib.as_array(eng.read_hidden())
    oh = np.ctypeslib.as_array(ctypes.cast(oracle.awqo_model_last_layer_out(model), ctypes.POINTER(ctypes.c_uint16)),
                               (cfg.hidden,))
    assert np.array_equal(hid, oh)
    lg = np.ctypeslib.as_array(eng.read_logits())
    ol = np.ctypeslib.as_array(ctypes.cast(oracle.awqo_model_logits(model), ctypes.POINTER(ctypes.c_uint16)),
                               (cfg.vocab,))
    assert np.array_equal(lg, ol)
    if n_prompt:
        eng.reset()
        eng.prefill(prompt.tolist())
        hs = np.ctypeslib.as_array(eng.read_hidden()).view(np.float16).astype(np.float32)
        eng.reset()
        eng.prefill(prompt.tolist(), batched=True)
        hb = np.ctypeslib.as_array(eng.read_hidden()).view(np.float16).astype(np.float32)
        assert np.isfinite(hs).all() and np.abs(hs - hb).max() <= 1e-2 * max(np.abs(hs).max(), 1e-6)
    eng.close()
    oracle.awqo_model_destroy(model)
