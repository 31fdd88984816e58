"""CPU pins of the oracle's composition functions.

awqo_model_layer (runOneLayer, Inference.cu:1029-1230), awqo_model_sample (sampleNextToken,
Inference.cu:1235-1292) and awqo_kv_append (Inference.cu:1094-1103) are compared bit for bit with a
second statement written here, in Python, straight from the reference's lines: the operator order,
which gamma each norm takes, what is rotated, where the cache rows go.  The arithmetic comes from the
oracle's primitives, each of which has its own pins in test_oracle_ops.py; the data movement (QKV
split, cache indexing) is numpy.  A mistake in the composition (gamma of another layer in the second
norm, rotary applied to V, a wrong head stride, residual taken from the wrong buffer) changes bits
here.
"""
import ctypes

import numpy as np
import pytest

from helpers import fill_pair, make_oracle_model, ptr, synth_normal


def _tensor(awq, oracle, model, layer, kind, part, dtype):
    nb = ctypes.c_int64(0)
    p = oracle.awqo_model_tensor(model, layer, kind, part, ctypes.byref(nb))
    n = nb.value // np.dtype(dtype).itemsize
    return np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(np.ctypeslib.as_ctypes_type(dtype))), (n,))


def _view_u16(p, n):
    return np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(ctypes.c_uint16)), (n,))


def _linear(oracle, w, m, k, x):
    y = np.zeros(m, dtype=np.uint16)
    oracle.awqo_linear(ptr(w[0]), ptr(w[1]), ptr(w[2]), m, k, ptr(x), ptr(y), 1)
    return y


def _rmsnorm(oracle, x, gamma, eps):
    out = np.zeros_like(x)
    oracle.awqo_rmsnorm(ptr(x), ptr(gamma), ptr(out), x.size, eps)
    return out


def _residual(oracle, a, b):
    out = np.zeros_like(a)
    oracle.awqo_residual(ptr(a), ptr(b), ptr(out), a.size)
    return out


def _setup(awq, oracle, seed, n_layers=3, hidden=512, inter=1536, vocab=1280, max_pos=24):
    cfg = awq.make_config(n_layers=n_layers, hidden=hidden, inter=inter, vocab=vocab, max_pos=max_pos)
    model = make_oracle_model(oracle, cfg)
    fill_pair(awq, oracle, cfg, seed, engine=None, model=model, profile=awq.SYNTH_BALANCED)
    return cfg, model


def _weights(awq, oracle, model, layer, kind):
    return [_tensor(awq, oracle, model, layer, kind, awq.P_PACKED, np.uint8),
            _tensor(awq, oracle, model, layer, kind, awq.P_SCALE, np.uint16),
            _tensor(awq, oracle, model, layer, kind, awq.P_ZP, np.uint16)]


def test_kv_append_is_head_major_row_copy(oracle):
    # Inference.cu:1094-1103: dst = cache + h*MAX_POS*HEAD_DIM + pos*HEAD_DIM, 128 halves per head
    n_heads, max_pos = 5, 11
    rng = np.random.default_rng(5)
    cache = rng.integers(0, 65536, n_heads * max_pos * 128, dtype=np.uint16)
    before = cache.copy()
    cur = rng.integers(0, 65536, n_heads * 128, dtype=np.uint16)
    for pos in (0, 7, max_pos - 1):
        oracle.awqo_kv_append(ptr(cache), ptr(cur), n_heads, max_pos, pos)
        want = before.reshape(n_heads, max_pos, 128)
        want[:, pos, :] = cur.reshape(n_heads, 128)
        assert np.array_equal(cache, want.reshape(-1)), pos
        before = cache.copy()


@pytest.mark.parametrize("layer,pos,L", [(0, 0, 1), (1, 5, 6), (2, 9, 9), (1, 23, 24)])
def test_model_layer_equals_the_reference_order_of_primitives(awq, oracle, layer, pos, L):
    cfg, model = _setup(awq, oracle, 4242)
    H, I, NH, MP = cfg.hidden, cfg.inter, cfg.hidden // 128, cfg.max_pos
    # state before the call: a seeded hidden vector and seeded cache rows at every position
    hidden = synth_normal(99, 1000 + layer, H).astype(np.float16).view(np.uint16)
    kc0 = (0.5 * synth_normal(99, 2000 + layer, NH * MP * 128)).astype(np.float16).view(np.uint16)
    vc0 = synth_normal(99, 3000 + layer, NH * MP * 128).astype(np.float16).view(np.uint16)
    _view_u16(oracle.awqo_model_hidden_mut(model), H)[:] = hidden
    _view_u16(oracle.awqo_model_kcache(model, layer), NH * MP * 128)[:] = kc0
    _view_u16(oracle.awqo_model_vcache(model, layer), NH * MP * 128)[:] = vc0

    oracle.awqo_model_layer(model, layer, pos, L)
    got_hidden = _view_u16(oracle.awqo_model_hidden(model), H).copy()
    got_kc = _view_u16(oracle.awqo_model_kcache(model, layer), NH * MP * 128).copy()
    got_vc = _view_u16(oracle.awqo_model_vcache(model, layer), NH * MP * 128).copy()

    # ---- second statement, by the reference's step numbers --------------------------------
    gamma = _tensor(awq, oracle, model, layer, awq.T_GAMMA, 0, np.uint16)
    cos_t = np.zeros(MP * 64, dtype=np.uint16)
    sin_t = np.zeros(MP * 64, dtype=np.uint16)
    oracle.awqo_rope_tables(ptr(cos_t), ptr(sin_t), MP)
    # 1) RMSNorm with this layer's gamma                                     Inference.cu:1035-1047
    normed = _rmsnorm(oracle, hidden, gamma, cfg.eps)
    # 2) Wqkv: m = 3H, k = H                                                 :1050-1066
    qkv = _linear(oracle, _weights(awq, oracle, model, layer, awq.T_WQKV), 3 * H, H, normed)
    # 3) split: Q = [0,H), K = [H,2H), V = [2H,3H); rotary on Q and K only   :1069-1091
    Q, K, V = qkv[:H].copy(), qkv[H:2 * H].copy(), qkv[2 * H:].copy()
    oracle.awqo_rotary(ptr(Q), ptr(cos_t), ptr(sin_t), NH, pos)
    oracle.awqo_rotary(ptr(K), ptr(cos_t), ptr(sin_t), NH, pos)
    # 4) cache[h][pos][:] = cur[h][:], head stride MAX_POS * 128            :1094-1103
    kc = kc0.copy().reshape(NH, MP, 128)
    vc = vc0.copy().reshape(NH, MP, 128)
    kc[:, pos, :] = K.reshape(NH, 128)
    vc[:, pos, :] = V.reshape(NH, 128)
    # 5) attention over L = current_seq_len_ + 1 positions                   :1106-1120
    ctx = np.zeros(H, dtype=np.uint16)
    oracle.awqo_attention(ptr(Q), ptr(kc), ptr(vc), ptr(ctx), NH, MP, L, None)
    # 6) Wo on the context, 7) hidden += attn_output                         :1123-1156
    attn = _linear(oracle, _weights(awq, oracle, model, layer, awq.T_WO), H, H, ctx)
    h1 = _residual(oracle, hidden, attn)
    # 8) RMSNorm of the updated hidden, the same gamma                       :1159-1170
    normed2 = _rmsnorm(oracle, h1, gamma, cfg.eps)
    # 9a) W1: m = I, k = H; 9b) GeLU in place; 9c) W2: m = H, k = I          :1174-1215
    mid = _linear(oracle, _weights(awq, oracle, model, layer, awq.T_W1), I, H, normed2)
    oracle.awqo_gelu(ptr(mid), I)
    mlp = _linear(oracle, _weights(awq, oracle, model, layer, awq.T_W2), H, I, mid)
    # 9d) hidden += mlp_output                                               :1217-1228
    h2 = _residual(oracle, h1, mlp)

    assert np.array_equal(got_kc, kc.reshape(-1))
    assert np.array_equal(got_vc, vc.reshape(-1))
    assert np.array_equal(got_hidden, h2)
    # the check has teeth: the layer changed the state, and the other layers' gammas differ
    assert not np.array_equal(got_hidden, hidden)
    other = _tensor(awq, oracle, model, (layer + 1) % cfg.n_layers, awq.T_GAMMA, 0, np.uint16)
    assert not np.array_equal(other, gamma)
    assert not np.array_equal(_rmsnorm(oracle, h1, other, cfg.eps), normed2)
    oracle.awqo_model_destroy(model)


def test_model_sample_is_norm_with_last_gamma_then_unembed_then_argmax(awq, oracle):
    cfg, model = _setup(awq, oracle, 777)
    H, V = cfg.hidden, cfg.vocab
    hidden = (3.0 * synth_normal(5, 77, H)).astype(np.float16).view(np.uint16)
    _view_u16(oracle.awqo_model_hidden_mut(model), H)[:] = hidden
    tok = oracle.awqo_model_sample(model)
    logits = _view_u16(oracle.awqo_model_logits(model), V).copy()
    # 1) RMSNorm with the LAST layer's gamma                                 Inference.cu:1243-1254
    gamma = _tensor(awq, oracle, model, cfg.n_layers - 1, awq.T_GAMMA, 0, np.uint16)
    normed = _rmsnorm(oracle, hidden, gamma, cfg.eps)
    # 2) unembedding: m = V, k = H, FP16 logits                              :1258-1274
    want = _linear(oracle, _weights(awq, oracle, model, 0, awq.T_UNEMBED), V, H, normed)
    assert np.array_equal(logits, want)
    # 3) strict > from index 0 over the logits widened to float              :1278-1290
    lf = want.view(np.float16).astype(np.float32)
    best, score = 0, lf[0]
    for i in range(1, V):
        if lf[i] > score:
            best, score = i, lf[i]
    assert tok == best == oracle.awqo_argmax(ptr(want), V)
    # the hidden state is not modified by sampling
    assert np.array_equal(_view_u16(oracle.awqo_model_hidden(model), H), hidden)
    # teeth: gamma of layer 0 would give other logits
    g0 = _tensor(awq, oracle, model, 0, awq.T_GAMMA, 0, np.uint16)
    assert not np.array_equal(_linear(oracle, _weights(awq, oracle, model, 0, awq.T_UNEMBED), V, H,
                                      _rmsnorm(oracle, hidden, g0, cfg.eps)), want)
    oracle.awqo_model_destroy(model)
