"""awq_decode_attention_static: the decode attention with its scratch (scores, part maxima, chunk sums,
chunk vectors) in a device array built into the library instead of a caller's workspace, for callers
that cannot allocate.  It must give the bits of awq_decode_attention (and so of the oracle), on calls in
a row that share the array: a long sequence, then shorter ones that leave most of the previous call's
scratch contents in place, across all launch forms (four, three, two launches and the one-workgroup
kernel that needs no scratch)."""
import ctypes

import numpy as np
import pytest

from helpers import ptr

pytestmark = pytest.mark.gpu


def test_static_scratch_attention_matches_the_workspace_entry_point(awq, lib, oracle, torch_gpu):
    torch = torch_gpu
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    nh, mp = 32, 9000            # the cache's capacity may exceed the 8192 positions the array is laid out for
    rng = np.random.default_rng(77)
    kc = (0.3 * rng.standard_normal((nh, mp, 128))).astype(np.float16)
    vc = rng.standard_normal((nh, mp, 128)).astype(np.float16)
    d_k, d_v = torch.from_numpy(kc).cuda(), torch.from_numpy(vc).cuda()
    ws = torch.zeros(lib.awq_attention_workspace_bytes(nh, mp), dtype=torch.uint8, device="cuda")
    for L in (8192, 3000, 1500, 700, 100, 2049, 1):   # each call after the first is smaller or another form
        q = rng.standard_normal(nh * 128).astype(np.float16)
        d_q = torch.from_numpy(q).cuda()
        want = torch.zeros(nh * 128, dtype=torch.float16, device="cuda")
        got = torch.full((nh * 128,), float("nan"), dtype=torch.float16, device="cuda")
        print("static-scratch attention, L", L, flush=True)
        awq.check(lib.awq_decode_attention(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), want.data_ptr(), nh, mp, L,
                                           ws.data_ptr(), st))
        awq.check(lib.awq_decode_attention_static(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), got.data_ptr(), nh,
                                                  mp, L, st))
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy().view(np.uint16), want.cpu().numpy().view(np.uint16)), L
        if L in (3000, 700):
            ref = np.zeros(nh * 128, dtype=np.float16)
            oracle.awqo_attention(ptr(q), ptr(kc), ptr(vc), ptr(ref), nh, mp, L, None)
            assert np.array_equal(got.cpu().numpy().view(np.uint16), ref.view(np.uint16)), L
    # fewer heads use a prefix of the same array
    q = rng.standard_normal(4 * 128).astype(np.float16)
    d_q = torch.from_numpy(q).cuda()
    want = torch.zeros(4 * 128, dtype=torch.float16, device="cuda")
    got = torch.zeros(4 * 128, dtype=torch.float16, device="cuda")
    awq.check(lib.awq_decode_attention(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), want.data_ptr(), 4, mp, 5000,
                                       ws.data_ptr(), st))
    awq.check(lib.awq_decode_attention_static(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), got.data_ptr(), 4, mp,
                                              5000, st))
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy().view(np.uint16), want.cpu().numpy().view(np.uint16))
    # beyond the array's size: refused, with a message
    assert lib.awq_decode_attention_static(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), got.data_ptr(), nh, mp, 8193,
                                           st) != 0
    assert b"8192" in lib.awq_last_error()
    assert lib.awq_decode_attention_static(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), got.data_ptr(), 33, mp, 10,
                                           st) != 0
    assert b"32 heads" in lib.awq_last_error()


def test_static_scratch_attention_allocates_nothing_and_can_be_captured(awq, lib, oracle, torch_gpu):
    """What the entry point is for: no device memory is allocated by any call after the first (which looks up
    the array's address), and a call issued under stream capture replays to the same bits."""
    torch = torch_gpu
    nh, mp = 32, 4096
    rng = np.random.default_rng(78)
    d_k = torch.from_numpy((0.3 * rng.standard_normal((nh, mp, 128))).astype(np.float16)).cuda()
    d_v = torch.from_numpy(rng.standard_normal((nh, mp, 128)).astype(np.float16)).cuda()
    d_q = torch.from_numpy(rng.standard_normal(nh * 128).astype(np.float16)).cuda()
    ws = torch.zeros(lib.awq_attention_workspace_bytes(nh, mp), dtype=torch.uint8, device="cuda")
    outs = {L: torch.zeros(nh * 128, dtype=torch.float16, device="cuda") for L in (3000, 1500, 900, 300)}
    wants = {L: torch.zeros(nh * 128, dtype=torch.float16, device="cuda") for L in outs}
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for L in outs:
        awq.check(lib.awq_decode_attention(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), wants[L].data_ptr(), nh, mp,
                                           L, ws.data_ptr(), st))
    # the first call on this device looks the array's address up
    awq.check(lib.awq_decode_attention_static(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), outs[300].data_ptr(), nh,
                                              mp, 300, st))
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        for L in outs:
            awq.check(lib.awq_decode_attention_static(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), outs[L].data_ptr(),
                                                      nh, mp, L, st))
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    for L in outs:
        assert torch.equal(outs[L].view(torch.int16), wants[L].view(torch.int16)), L
    # under stream capture: every launch form, replayed three times with eager work in between
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    cap = {L: torch.zeros(nh * 128, dtype=torch.float16, device="cuda") for L in outs}
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        cst = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for L in outs:
            awq.check(lib.awq_decode_attention_static(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), cap[L].data_ptr(),
                                                      nh, mp, L, cst))
    for replay in range(3):
        for L in outs:
            cap[L].fill_(float("nan"))
        torch.cuda.synchronize()
        print("replay", replay, flush=True)
        graph.replay()
        torch.cuda.synchronize()
        for L in outs:
            assert torch.equal(cap[L].view(torch.int16), wants[L].view(torch.int16)), (replay, L)
