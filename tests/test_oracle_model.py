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


def test_block_fixed_point_products_against_the_reference_arithmetic_on_the_whole_model(awq, oracle):
    """The linear layers of the GPU path (and of awqo_linear) put each block of 32 inputs into 16-bit block
    fixed point and apply scale and zero-point to exact integer block sums; the reference multiplies
    binary16-rounded weights h(h(q-z)*s) (Inference.cu:102-104) and accumulates in binary32
    (awqo_linear_seq).  Per product the two agree to about 1e-3 of the output's rms (test_oracle_ops.py);
    here the distance is measured on the whole 36-layer model at the reference widths: the same prompt runs
    once with each arithmetic in every linear layer, and the last layer's output, the last logits and the
    greedy ids are compared.  Measured: largest logit difference 6.3e-3 (logit std 0.94, i.e. 0.7 %), largest
    hidden difference 0.44 (rms 66, 0.7 %), ids identical; the bounds below leave a factor of three."""
    cfg = awq.make_config(max_pos=16)
    assert (cfg.n_layers, cfg.hidden, cfg.inter, cfg.vocab) == (36, 4096, 12288, 151936)
    model = make_oracle_model(oracle, cfg)
    fill_pair(awq, oracle, cfg, 2025, engine=None, model=model, profile=awq.SYNTH_BALANCED)
    prompt = np.zeros(4, dtype=np.int32)
    awq.check(awq.load_library().awq_synth_tokens(2025, awq.SYNTH_STREAM_INPUT, ptr(prompt), 4, cfg.vocab))
    N = 4
    runs = {}
    for mode in (0, 1):
        oracle.awqo_model_set_linear_mode(model, mode)
        out = np.zeros(N, dtype=np.int32)
        assert oracle.awqo_model_generate(model, ptr(prompt), prompt.size, N, ptr(out)) == N
        logits = np.ctypeslib.as_array(ctypes.cast(oracle.awqo_model_logits(model), ctypes.POINTER(ctypes.c_uint16)),
                                       (cfg.vocab,)).copy().view(np.float16).astype(np.float64)
        hidden = np.ctypeslib.as_array(ctypes.cast(oracle.awqo_model_last_layer_out(model),
                                                   ctypes.POINTER(ctypes.c_uint16)),
                                       (cfg.hidden,)).copy().view(np.float16).astype(np.float64)
        margins = np.zeros(N, dtype=np.float32)
        assert oracle.awqo_model_margins(model, ptr(margins), N) == N
        runs[mode] = (out.tolist(), logits, hidden, margins.copy())
    oracle.awqo_model_set_linear_mode(model, 0)
    oracle.awqo_model_destroy(model)
    (ids_b, lg_b, hid_b, mg_b), (ids_r, lg_r, hid_r, mg_r) = runs[0], runs[1]
    assert np.isfinite(lg_r).all() and np.isfinite(lg_b).all()
    d_logit = np.abs(lg_b - lg_r).max()
    d_hidden = np.abs(hid_b - hid_r).max()
    print("logits: largest difference %.4g, std %.4g; hidden: largest difference %.4g, rms %.4g; ids %s / %s"
          % (d_logit, lg_r.std(), d_hidden, np.sqrt((hid_r ** 2).mean()), ids_b, ids_r))
    assert d_logit <= 2e-2 * lg_r.std()
    assert d_hidden <= 2e-2 * np.sqrt((hid_r ** 2).mean())
    assert d_logit > 0 or d_hidden > 0          # the two arithmetics are different ones
    # an id may only differ where the reference arithmetic's own top-1/top-2 margin is within the drift
    for step, (a, b) in enumerate(zip(ids_b, ids_r)):
        if a != b:
            assert mg_r[step] <= 2 * d_logit + 2.0 ** -6, (step, a, b, mg_r[step])
            break  # after a differing id the two runs see different inputs
    assert len(set(ids_r)) > 1
