"""Batched prompt pass (all prompt positions through each layer together, products on the matrix
cores) against the token-by-token prompt loop and the CPU oracle.

The two prompt loops sum the products in different orders, so their states agree to binary16
rounding noise (tolerance below), not bit for bit; greedy tokens must be identical except where the
oracle's own top-1/top-2 logit margin is within that noise."""
import ctypes

import numpy as np
import pytest

from helpers import fill_pair, make_oracle_model, ptr

pytestmark = pytest.mark.gpu

SMALL = dict(n_layers=4, hidden=512, inter=1536, vocab=1024, max_pos=160)
REL_TOL = 1e-2      # of the largest magnitude of the vector compared
MARGIN_TOL = 0.05   # logit units: a flip is only acceptable below this top-1/top-2 margin


def as_f32(u16):
    return np.ctypeslib.as_array(u16).view(np.float16).astype(np.float32)


def close(a, b):
    return np.abs(a - b).max() <= REL_TOL * max(np.abs(a).max(), 1e-6)


def check_tokens(got, ref, margins, what):
    for i, (g, r) in enumerate(zip(got, ref)):
        if g != r:
            assert margins[i] < MARGIN_TOL, "%s: token %d differs (%d vs %d) at margin %.4f" % (what, i, g, r, margins[i])
            return i       # sequences diverge legitimately after a tie-like step
    return len(ref)


def oracle_run(oracle, model, prompt, n_new):
    p = np.asarray(prompt, dtype=np.int32)
    out = np.zeros(max(1, n_new), dtype=np.int32)
    assert oracle.awqo_model_generate(model, ptr(p), p.size, n_new, ptr(out)) == n_new
    margins = np.zeros(max(1, n_new), dtype=np.float32)
    oracle.awqo_model_margins(model, ptr(margins), n_new)
    return out[:n_new].tolist(), margins


# hidden 4096 and an intermediate size of 8192: the products of a prompt of 2..16 tokens go to the kernel for
# up to 16 tokens (k a multiple of 4096) with its residual and GeLU endings, one and two slices of k
WIDE = dict(n_layers=2, hidden=4096, inter=8192, vocab=1024, max_pos=64)
# the reference's widths: a prompt of 17..64 tokens takes the kernels that share the token tiles through LDS, with
# their store, residual and GeLU endings (16 and 64 rows per workgroup, one token tile and two); one of 150 tokens
# takes them 64 tokens at a time, and the 4096 x 12288 product with k cut over four workgroups
FULLW = dict(n_layers=2, hidden=4096, inter=12288, vocab=1024, max_pos=192)


@pytest.mark.parametrize("shape,n_prompt", [(SMALL, 1), (SMALL, 2), (SMALL, 5), (SMALL, 37), (SMALL, 100),
                                            (WIDE, 3), (WIDE, 12), (WIDE, 16), (WIDE, 20), (WIDE, 40),
                                            (FULLW, 24), (FULLW, 50), (FULLW, 150)],
                         ids=lambda v: ("hidden%d-inter%d" % (v["hidden"], v["inter"])) if isinstance(v, dict) else str(v))
def test_small_model_batched_prompt_matches_sequential(awq, oracle, torch_gpu, shape, n_prompt):
    cfg = awq.make_config(**shape)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 77, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    rng = np.random.default_rng(n_prompt)
    prompt = rng.integers(0, cfg.vocab, n_prompt).tolist()
    n_new = 16
    print("batched prompt pass, small model, P =", n_prompt, flush=True)

    eng.reset()
    eng.prefill(prompt)
    hid_seq = as_f32(eng.read_hidden()).copy()
    tok_seq = eng.decode(n_new)

    eng.reset()
    eng.prefill(prompt, batched=True)
    hid_bat = as_f32(eng.read_hidden()).copy()
    tok_bat = eng.decode(n_new)

    assert np.isfinite(hid_seq).all() and np.abs(hid_seq).max() > 0
    assert close(hid_seq, hid_bat)
    ref, margins = oracle_run(oracle, model, prompt, n_new)
    assert tok_seq == ref                      # the sequential loop is bit-exact with the oracle
    same = check_tokens(tok_bat, ref, margins, "batched")
    print("identical tokens: %d of %d; min margin %.4f" % (same, n_new, margins.min()), flush=True)

    # generateResponse honours the mode switch
    eng.set_prefill_mode(True)
    assert eng.generateResponse(prompt, n_new) == tok_bat
    eng.set_prefill_mode(False)
    assert eng.generateResponse(prompt, n_new) == ref
    eng.close()
    oracle.awqo_model_destroy(model)


def test_batched_prompt_in_pieces_equals_one_call(awq, oracle, torch_gpu):
    """Positions, attended lengths and cache rows must not depend on how the prompt is cut into
    calls.  The pieces are long enough (more than 32 tokens) for the same product kernel to serve
    them and the whole prompt, and that kernel's result for a token does not depend on the other
    tokens, so the state is bit-identical."""
    cfg = awq.make_config(**SMALL)
    model = make_oracle_model(oracle, cfg)   # only as the host buffer of the weights here
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 78, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    oracle.awqo_model_destroy(model)
    rng = np.random.default_rng(5)
    prompt = rng.integers(0, cfg.vocab, 90).tolist()
    print("batched prompt pass in pieces", flush=True)
    eng.reset()
    eng.prefill(prompt, batched=True)
    whole = np.ctypeslib.as_array(eng.read_hidden()).copy()
    tok_whole = eng.decode(8)
    eng.reset()
    eng.prefill(prompt[:41], batched=True)
    eng.prefill(prompt[41:], batched=True)
    pieces = np.ctypeslib.as_array(eng.read_hidden()).copy()
    assert np.array_equal(whole, pieces)
    assert eng.decode(8) == tok_whole
    # a sequential start followed by a batched rest stays within rounding noise of it
    eng.reset()
    eng.prefill(prompt[:7])
    eng.prefill(prompt[7:], batched=True)
    mixed = np.ctypeslib.as_array(eng.read_hidden()).copy()
    assert close(whole.view(np.float16).astype(np.float32), mixed.view(np.float16).astype(np.float32))
    # error paths: prompt tokens after generated ones, an id outside the vocabulary, overflow of max_pos
    eng.decode(1)
    with pytest.raises(awq.AwqError):
        eng.prefill([1], batched=True)
    eng.reset()
    with pytest.raises(awq.AwqError):
        eng.prefill([cfg.vocab], batched=True)
    with pytest.raises(awq.AwqError):
        eng.prefill([1] * (cfg.max_pos + 1), batched=True)
    eng.prefill([], batched=True)
    eng.close()


def test_full_model_batched_prompt_tokens(awq, oracle, torch_gpu):
    """36 layers at full width, 128-token prompt: the tokens after a batched prompt pass are the
    oracle's."""
    cfg = awq.make_config(max_pos=192)
    model = make_oracle_model(oracle, cfg)
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 2024, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    lib = awq.load_library()
    prompt = np.zeros(128, dtype=np.int32)
    awq.check(lib.awq_synth_tokens(2024, awq.SYNTH_STREAM_INPUT, ptr(prompt), prompt.size, cfg.vocab))
    n_new = 32
    print("batched prompt pass, full model, P = 128", flush=True)
    eng.reset()
    eng.prefill(prompt.tolist(), batched=True)
    hid_bat = as_f32(eng.read_hidden()).copy()
    tok_bat = eng.decode(n_new)
    eng.reset()
    eng.prefill(prompt.tolist())
    hid_seq = as_f32(eng.read_hidden()).copy()
    tok_seq = eng.decode(n_new)
    print("hidden: max |seq - batched| = %.5f at scale %.3f" % (np.abs(hid_seq - hid_bat).max(), np.abs(hid_seq).max()),
          flush=True)
    assert close(hid_seq, hid_bat)
    ref, margins = oracle_run(oracle, model, prompt.tolist(), n_new)
    assert tok_seq == ref
    same = check_tokens(tok_bat, ref, margins, "batched")
    print("identical tokens: %d of %d; min margin %.4f" % (same, n_new, margins.min()), flush=True)
    # A differing id is acceptable only at a step where the oracle's own margin is below MARGIN_TOL (checked
    # above) and for that reason only: the logits the batched run sampled that id from must be the oracle's
    # to rounding noise.  Compared at the first differing step, or at the last step when all ids agree.
    d = min(same, n_new - 1)
    ref_d, _ = oracle_run(oracle, model, prompt.tolist(), d + 1)
    assert ref_d == ref[:d + 1]
    lg_ref = np.ctypeslib.as_array(ctypes.cast(oracle.awqo_model_logits(model), ctypes.POINTER(ctypes.c_uint16)),
                                   (cfg.vocab,)).copy().view(np.float16).astype(np.float32)
    eng.reset()
    eng.prefill(prompt.tolist(), batched=True)
    assert eng.decode(d + 1) == tok_bat[:d + 1]
    lg_bat = as_f32(eng.read_logits()).copy()
    print("logits at step %d: max |oracle - batched| = %.5f at scale %.3f" %
          (d, np.abs(lg_ref - lg_bat).max(), np.abs(lg_ref).max()), flush=True)
    assert np.isfinite(lg_bat).all() and close(lg_ref, lg_bat)
    eng.close()
    oracle.awqo_model_destroy(model)


def test_long_prompt_takes_the_rows_split_products(awq, oracle, torch_gpu):
    """A 1027-token prompt at full width: every product of the layer has enough output tiles for the
    rows-split workgroup shapes (Wqkv and W1 a tile per workgroup, Wo and W2 with their 144 tiles cut
    evenly over 256 workgroups that hand FP32 sums over; GeLU and residual epilogues), and the prompt
    spans the short-sequence and the long-sequence attention launches of the batched pass."""
    cfg = awq.make_config(n_layers=1, vocab=2048, max_pos=1100)
    model = make_oracle_model(oracle, cfg)   # only as the host buffer of the weights here
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 31, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    oracle.awqo_model_destroy(model)
    rng = np.random.default_rng(9)
    prompt = rng.integers(0, cfg.vocab, 1027).tolist()
    print("batched prompt pass, one full-width layer, P = 1027", flush=True)
    eng.reset()
    eng.prefill(prompt)
    hid_seq = as_f32(eng.read_hidden()).copy()
    tok_seq = eng.decode(4)
    eng.reset()
    eng.prefill(prompt, batched=True)
    hid_bat = as_f32(eng.read_hidden()).copy()
    tok_bat = eng.decode(4)
    print("hidden: max |seq - batched| = %.5f at scale %.3f" % (np.abs(hid_seq - hid_bat).max(), np.abs(hid_seq).max()),
          flush=True)
    assert np.isfinite(hid_seq).all() and close(hid_seq, hid_bat)
    assert tok_bat[0] == tok_seq[0]
    eng.close()


def test_maximum_sequence_length_one_layer(awq, oracle, torch_gpu):
    """The reference's MAX_POSITION_EMBEDDINGS (40960, Inference.cu:39) on one full-width layer: a
    40,950-token prompt through the batched pass and, token by token, through the bit-exact decode
    kernels (attention cut along the sequence beyond 704 positions), then generation up to the
    last position; one more token is an error, not a cache overrun."""
    cfg = awq.make_config(n_layers=1, vocab=2048, max_pos=40960)
    model = make_oracle_model(oracle, cfg)   # only as the host buffer of the weights here
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 40, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    oracle.awqo_model_destroy(model)
    rng = np.random.default_rng(40960)
    prompt = rng.integers(0, cfg.vocab, 40950).tolist()
    print("maximum sequence length: batched prompt pass", flush=True)
    eng.reset()
    eng.prefill(prompt, batched=True)
    hid_bat = as_f32(eng.read_hidden()).copy()
    tok_bat = eng.decode(10)            # positions 40950 .. 40959
    with pytest.raises(awq.AwqError):
        eng.decode(1)
    print("maximum sequence length: token by token", flush=True)
    eng.reset()
    eng.prefill(prompt)
    hid_seq = as_f32(eng.read_hidden()).copy()
    tok_seq = eng.decode(10)
    print("hidden: max |seq - batched| = %.5f at scale %.3f; tokens %s / %s" %
          (np.abs(hid_seq - hid_bat).max(), np.abs(hid_seq).max(), tok_seq, tok_bat), flush=True)
    assert np.isfinite(hid_seq).all() and close(hid_seq, hid_bat)
    assert tok_seq[0] == tok_bat[0]
    with pytest.raises(awq.AwqError):
        eng.generateResponse(prompt, 11)   # 40950 + 11 > 40960
    eng.close()


def test_handed_over_sums_give_up_path(awq, lib, oracle, torch_gpu):
    """Some products of the batched pass cut their work evenly over the workgroups and hand FP32 partial sums to
    the workgroup that holds a tile's last steps, which waits for them (bounded).  The give-up path of that
    wait, driven from the host: with the "give up now" word set, every such wait ends before its first poll,
    every kernel runs to its end, the status word reports it, and the workgroups that gave up leave their
    tiles unwritten.  Through the kernel entry point first, then through the engine, which must return an
    error and work again after awq_reset."""
    torch = torch_gpu
    import ctypes as C
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    m, k, M = 4096, 12288, 1024
    assert lib.awq_gemm_plan(m, k, M, 1) == 4          # rows split, work cut evenly, sums handed over
    rng = np.random.default_rng(12)
    packed = rng.integers(0, 256, size=m * k // 2, dtype=np.uint8)
    scale = rng.uniform(0.002, 0.02, size=m // 128).astype(np.float16)
    zp = rng.integers(0, 16, size=m // 128).astype(np.float16)
    x = rng.standard_normal((M, k)).astype(np.float16)
    d_in = torch.from_numpy(packed).cuda()
    d_w = torch.zeros_like(d_in)
    awq.check(lib.awq_linear_repack(d_in.data_ptr(), d_w.data_ptr(), m, k, st))
    d_s, d_z, d_x = torch.from_numpy(scale).cuda(), torch.from_numpy(zp).cuda(), torch.from_numpy(x).cuda()
    d_ws = torch.zeros(lib.awq_gemm_workspace_bytes(m, k, M), dtype=torch.uint8, device="cuda")
    head = d_ws[:4096].view(torch.int32)

    def product():
        y = torch.full((M, m), float("nan"), dtype=torch.float16, device="cuda")
        awq.check(lib.awq_gemm(d_w.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), m, k, d_x.data_ptr(), y.data_ptr(), M, 1,
                               d_ws.data_ptr(), st))
        torch.cuda.synchronize()
        return y

    print("product with handed-over sums", flush=True)
    good = product()
    assert int(head[0].item()) == 0 and bool(torch.isfinite(good).all())
    print("the same with the give-up word set", flush=True)
    head[1] = 1
    bad = product()
    assert int(head[0].item()) == 1                     # reported
    unwritten = torch.isnan(bad)
    assert bool(unwritten.any())                        # the tiles of the workgroups that gave up
    assert bool((bad[~unwritten] == good[~unwritten]).all())  # nothing half-summed was stored
    d_ws[:4096] = 0                                     # what the header asks for after a give-up
    again = product()
    assert int(head[0].item()) == 0 and bool((again == good).all())

    # the engine: a 640-token prompt on one full-width layer sends W2 through the same kernel
    cfg = awq.make_config(n_layers=1, vocab=2048, max_pos=704)
    model = make_oracle_model(oracle, cfg)   # only as the host buffer of the weights here
    eng = awq.QWen3AWQInfer.empty(cfg)
    fill_pair(awq, oracle, cfg, 32, engine=eng, model=model, profile=awq.SYNTH_BALANCED)
    oracle.awqo_model_destroy(model)
    prompt = rng.integers(0, cfg.vocab, 640).tolist()
    assert lib.awq_gemm_plan(cfg.hidden, cfg.inter, 640, 1) == 4
    print("engine: batched prompt pass", flush=True)
    eng.reset()
    eng.prefill(prompt, batched=True)
    hid = np.ctypeslib.as_array(eng.read_hidden()).copy()
    tok = eng.decode(4)
    print("engine: the same with every hand-over giving up", flush=True)
    eng.reset()
    awq.check(lib.awq_debug_force_handover_giveup(eng._h, 1))
    with pytest.raises(awq.AwqError) as ei:
        eng.prefill(prompt, batched=True)
    assert ei.value.code == 3 and "gave up" in str(ei.value)
    print("engine: and again after a reset", flush=True)
    eng.reset()
    eng.prefill(prompt, batched=True)
    assert np.array_equal(np.ctypeslib.as_array(eng.read_hidden()), hid)
    assert eng.decode(4) == tok
    eng.close()
