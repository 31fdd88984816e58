"""The oracle's transcription of the host loop (generateResponse, Inference.cu:1297-1408) against
a second, independent statement of the same schedule written in Python on top of the oracle's
single-layer primitives."""
import ctypes

import numpy as np
import pytest

from helpers import fill_pair, make_oracle_model, ptr


def expected_schedule(P, N, n_layers, split):
    """(layer, pos, attended length) of every runOneLayer call, derived by hand from the reference:
    current_seq_len_ starts at 0 (I:430); the prompt loop sets it to t after *each* layer
    (I:1331, 1341); generation sets it to pos after the first `split` layers (I:1364);
    attention uses current_seq_len_ + 1 (I:1118)."""
    calls, csl = [], 0
    for t in range(P):
        for l in range(n_layers):
            calls.append((l, t, csl + 1))
            csl = t
    for step in range(N):
        pos = P + step
        for l in range(split):
            calls.append((l, pos, csl + 1))
        csl = pos
        for l in range(split, n_layers):
            calls.append((l, pos, csl + 1))
    return calls


def test_schedule_table():
    # the quirks spelled out: layer 0 of prompt token t >= 1 attends t positions (not t+1), and in
    # generation the first half of the layers does not see the current position
    s = expected_schedule(3, 2, 4, 2)
    assert s[:4] == [(0, 0, 1), (1, 0, 1), (2, 0, 1), (3, 0, 1)]
    assert s[4:8] == [(0, 1, 1), (1, 1, 2), (2, 1, 2), (3, 1, 2)]
    assert s[8:12] == [(0, 2, 2), (1, 2, 3), (2, 2, 3), (3, 2, 3)]
    assert s[12:16] == [(0, 3, 3), (1, 3, 3), (2, 3, 4), (3, 3, 4)]
    assert s[16:20] == [(0, 4, 4), (1, 4, 4), (2, 4, 5), (3, 4, 5)]


@pytest.mark.parametrize("P,N", [(0, 3), (1, 4), (5, 6)])
def test_generate_follows_the_schedule(awq, oracle, P, N):
    cfg = awq.make_config(n_layers=4, hidden=512, inter=512, vocab=1024, max_pos=32, split_idx=2)
    model = make_oracle_model(oracle, cfg)
    fill_pair(awq, oracle, cfg, 31337, engine=None, model=model)
    prompt = np.array([(7 * i + 3) % cfg.vocab for i in range(P)], dtype=np.int32)
    out = np.zeros(max(N, 1), dtype=np.int32)
    assert oracle.awqo_model_generate(model, ptr(prompt) if P else None, P, N, ptr(out)) == N
    ref_tokens = out[:N].tolist()
    final_hidden = np.ctypeslib.as_array(ctypes.cast(oracle.awqo_model_hidden(model), ctypes.POINTER(ctypes.c_uint16)),
                                         (cfg.hidden,)).copy()

    # second statement: drive the layer primitive by the hand-derived schedule
    oracle.awqo_model_reset(model)
    nb = ctypes.c_int64(0)
    emb = [oracle.awqo_model_tensor(model, 0, awq.T_EMBED, part, ctypes.byref(nb)) for part in range(3)]
    hid = oracle.awqo_model_hidden_mut(model)

    def embed(tok):
        oracle.awqo_embed(emb[0], emb[1], emb[2], cfg.hidden, cfg.vocab, tok, hid)

    sched = expected_schedule(P, N, cfg.n_layers, cfg.split_idx)
    it = iter(sched)
    for t in range(P):
        embed(int(prompt[t]))
        for _ in range(cfg.n_layers):
            l, pos, L = next(it)
            oracle.awqo_model_layer(model, l, pos, L)
    toks = []
    for step in range(N):
        for _ in range(cfg.n_layers):
            l, pos, L = next(it)
            oracle.awqo_model_layer(model, l, pos, L)
        tok = oracle.awqo_model_sample(model)
        toks.append(tok)
        embed(tok)
    assert toks == ref_tokens
    hidden2 = np.ctypeslib.as_array(ctypes.cast(oracle.awqo_model_hidden(model), ctypes.POINTER(ctypes.c_uint16)),
                                    (cfg.hidden,))
    assert np.array_equal(final_hidden, hidden2)
    assert oracle.awqo_model_generate(model, ptr(prompt) if P else None, P, cfg.max_pos - P + 1, ptr(out)) == -1
    oracle.awqo_model_destroy(model)
