"""GPU parity: every HIP kernel, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Integer / FP16-rounded outputs must match bit for bit; the fused linear kernel is
also held to 1e-2 relative against the plain sequential FP32-accumulate product."""
import ctypes

import numpy as np
import pytest

from helpers import bits16, f16, ptr, repack_numpy

pytestmark = pytest.mark.gpu


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def stream(torch):
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def rand_awq(rng, m, k, n_groups=None, zp_int=True):
    n_groups = n_groups or m // 128
    packed = rng.integers(0, 256, size=m * k // 2, dtype=np.uint8)
    scale = rng.uniform(0.002, 0.02, size=n_groups).astype(np.float16)
    zp = (rng.integers(0, 16, size=n_groups) if zp_int else rng.uniform(0, 15, size=n_groups)).astype(np.float16)
    return packed, scale, zp


# ----------------------------------------------------------------------------- dequant
@pytest.mark.parametrize("rows,cols,ng,zp_int", [(4096, 4096, 32, True), (384, 1024, 3, False), (128, 151936 // 8, 1, True)])
def test_dequant_bit_exact(awq, lib, oracle, torch_gpu, rows, cols, ng, zp_int):
    torch = torch_gpu
    rng = np.random.default_rng(rows + cols)
    packed = rng.integers(0, 256, size=rows * cols // 2, dtype=np.uint8)
    scale = rng.uniform(0.002, 0.02, size=ng).astype(np.float16)
    zp = (rng.integers(0, 16, size=ng) if zp_int else rng.uniform(0, 15, size=ng)).astype(np.float16)
    ref = np.zeros(rows * cols, dtype=np.float16)
    oracle.awqo_dequant(ptr(packed), ptr(scale), ptr(zp), ptr(ref), rows, cols, ng)
    d_p, d_s, d_z = dev(torch, packed), dev(torch, scale), dev(torch, zp)
    d_o = torch.zeros(rows * cols, dtype=torch.float16, device="cuda")
    awq.check(lib.awq_dequant(d_p.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), d_o.data_ptr(), rows, cols, ng,
                              stream(torch)))
    torch.cuda.synchronize()
    got = d_o.cpu().numpy()
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


def test_dequant_special_scale_zp_patterns(awq, lib, oracle, torch_gpu):
    torch = torch_gpu
    scales = np.concatenate([f16(np.arange(0x1800, 0x2600, 7, dtype=np.uint16)),
                             f16(np.array([0x0001, 0x03ff, 0x0400, 0x3c00, 0x3555, 0x7bff], dtype=np.uint16))])
    zps = np.concatenate([np.arange(16).astype(np.float16), f16(np.arange(0x3c00, 0x4b80, 97, dtype=np.uint16)),
                          np.array([0.5, 7.25, 1e-4, 1023.0, -3.0], dtype=np.float16)])
    S, Z = np.meshgrid(scales, zps, indexing="ij")
    S, Z = np.ascontiguousarray(S.reshape(-1)), np.ascontiguousarray(Z.reshape(-1))
    n = S.size
    cols = 128 * n
    nib = (np.arange(cols) % 16).astype(np.uint8)
    packed = (nib[0::2] | (nib[1::2] << 4)).astype(np.uint8)
    ref = np.zeros(cols, dtype=np.float16)
    oracle.awqo_dequant(ptr(packed), ptr(S), ptr(Z), ptr(ref), 1, cols, n)
    d_o = torch.zeros(cols, dtype=torch.float16, device="cuda")
    d_p, d_s, d_z = dev(torch, packed), dev(torch, S), dev(torch, Z)
    awq.check(lib.awq_dequant(d_p.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), d_o.data_ptr(), 1, cols, n, stream(torch)))
    torch.cuda.synchronize()
    assert np.array_equal(d_o.cpu().numpy().view(np.uint16), ref.view(np.uint16))


# ----------------------------------------------------------------------------- repack + fused linear
@pytest.mark.parametrize("m,k", [(128, 512), (384, 512), (256, 1024)])
def test_repack_matches_numpy_layout(awq, lib, oracle, torch_gpu, m, k):
    torch = torch_gpu
    rng = np.random.default_rng(m * 7 + k)
    packed = rng.integers(0, 256, size=m * k // 2, dtype=np.uint8)
    C = oracle.awqo_group_period(m, k)
    ref = repack_numpy(packed, m, k, C)
    d_in = dev(torch, packed)
    d_out = torch.zeros(m * k // 2, dtype=torch.uint8, device="cuda")
    awq.check(lib.awq_linear_repack(d_in.data_ptr(), d_out.data_ptr(), m, k, stream(torch)))
    torch.cuda.synchronize()
    assert np.array_equal(d_out.cpu().numpy().view(np.uint32), ref)


def gemv_gpu(awq, lib, torch, packed, scale, zp, m, k, x, repeat=1):
    d_in = dev(torch, packed)
    d_w = torch.zeros(m * k // 2, dtype=torch.uint8, device="cuda")
    awq.check(lib.awq_linear_repack(d_in.data_ptr(), d_w.data_ptr(), m, k, stream(torch)))
    d_s, d_z, d_x = dev(torch, scale), dev(torch, zp), dev(torch, x)
    ws = torch.zeros(lib.awq_gemv_workspace_bytes(m, k), dtype=torch.uint8, device="cuda")
    outs = []
    for _ in range(repeat):
        d_y = torch.full((m,), float("nan"), dtype=torch.float16, device="cuda")
        awq.check(lib.awq_gemv(d_w.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), m, k, d_x.data_ptr(), d_y.data_ptr(),
                               ws.data_ptr(), stream(torch)))
        torch.cuda.synchronize()
        outs.append(d_y.cpu().numpy())
    assert int(ws.to(torch.int32).abs().sum().item()) == 0  # the workspace is left zeroed
    return outs


# (512, 8192), (1024, 16384): few rows and long k, where a workgroup takes half a row group (general and
# 16-wavefront forms); the last two: more than 1024 row groups, several per workgroup
GEMV_SHAPES = [(128, 512), (256, 1024), (384, 512), (128, 1536), (640, 2048), (4096, 4096), (12288, 4096),
               (4096, 12288), (512, 8192), (1024, 16384), (20480, 1024), (40960, 512)]


@pytest.mark.parametrize("m,k", GEMV_SHAPES)
@pytest.mark.parametrize("zp_int", [True, False])
def test_gemv_bit_exact_and_within_tolerance(awq, lib, oracle, torch_gpu, m, k, zp_int):
    torch = torch_gpu
    rng = np.random.default_rng(m * 31 + k + int(zp_int))
    packed, scale, zp = rand_awq(rng, m, k, zp_int=zp_int)
    x = rng.standard_normal(k).astype(np.float16)
    ref = np.zeros(m, dtype=np.float16)
    oracle.awqo_linear(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(x), ptr(ref), 1)
    seq = np.zeros(m, dtype=np.float16)
    oracle.awqo_linear_seq(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(x), ptr(seq), 1)
    outs = gemv_gpu(awq, lib, torch, packed, scale, zp, m, k, x, repeat=2)
    print("gemv", m, k, zp_int, flush=True)
    assert np.array_equal(outs[0].view(np.uint16), ref.view(np.uint16))          # same summation order: same bits
    assert np.array_equal(outs[1].view(np.uint16), ref.view(np.uint16))          # and the workspace reset itself
    # against plain sequential FP32 accumulation of the binary16-dequantised weights: 1e-2 relative (north
    # star tolerance); outputs smaller than the root mean square of all outputs are measured against that.
    # The kernel applies scale and zero-point to block sums, so it differs from this reference by the
    # binary16 rounding of the weights: 99% of the outputs within 2^-9 of that scale.
    want = seq.astype(np.float64)
    denom = np.maximum(np.abs(want), np.sqrt(np.mean(want * want)))
    err = np.abs(outs[0].astype(np.float64) - want) / denom
    assert np.all(err <= 1e-2) and np.percentile(err, 99) <= 2.0 ** -9


@pytest.mark.parametrize("m,k", [(4096, 4096), (12288, 4096), (4096, 12288)])
def test_gemv_heavy_tailed_inputs_stay_within_tolerance(awq, lib, oracle, torch_gpu, m, k):
    """outliers, massive channels, heavy tails and post-GeLU inputs at the model's own matrix shapes: the fused
    product must still give the oracle's bits, and stay within 1e-2 of max(|y|, rms y) of the plain
    FP32-accumulate product over the reference's binary16-rounded weights (awqo_linear_seq); the block fixed
    point rounds each input to 2^-16 of its block's largest magnitude, so the distance depends on the shape
    of x"""
    from helpers import heavy_tailed_inputs
    torch = torch_gpu
    rng = np.random.default_rng(m + 3 * k)
    packed, scale, zp = rand_awq(rng, m, k)
    for name, x in heavy_tailed_inputs(rng, k).items():
        ref = np.zeros(m, dtype=np.float16)
        oracle.awqo_linear(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(x), ptr(ref), 1)
        seq = np.zeros(m, dtype=np.float16)
        oracle.awqo_linear_seq(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(x), ptr(seq), 1)
        got = gemv_gpu(awq, lib, torch, packed, scale, zp, m, k, x)[0]
        print("gemv", m, k, name, flush=True)
        assert np.array_equal(got.view(np.uint16), ref.view(np.uint16)), name
        want = seq.astype(np.float64)
        if not np.isfinite(want).all():
            assert np.array_equal(np.isfinite(want), np.isfinite(got.astype(np.float64))), name
            continue
        denom = np.maximum(np.abs(want), np.sqrt(np.mean(want * want)))
        err = np.abs(got.astype(np.float64) - want) / denom
        assert err.max() <= 1e-2, (name, err.max())


@pytest.mark.parametrize("m,k", [(256, 1024), (384, 512), (4096, 4096), (128 * 37, 512)])
def test_gemv_input_dynamic_range(awq, lib, oracle, torch_gpu, m, k):
    """the inputs' block fixed point at its corners: subnormal and zero blocks, inputs far below their
    block's largest, the largest binary16 values, and blocks that hold an infinity or a NaN"""
    torch = torch_gpu
    rng = np.random.default_rng(m + 7 * k)
    packed, scale, zp = rand_awq(rng, m, k, zp_int=False)
    x = rng.standard_normal(k).astype(np.float16)
    x[0:32] = 0                                                     # a block of zeros (one of them negative)
    x[5] = np.float16(-0.0)
    x[32:64] = (rng.integers(-1023, 1024, 32).astype(np.float64) * 2.0 ** -24).astype(np.float16)   # subnormals only
    x[64:96] *= np.float16(2.0 ** -12)                              # small normals and subnormals mixed
    x[96:128] = np.clip(rng.standard_normal(32) * 20000, -65504, 65504).astype(np.float16)  # up to the top of the range
    x[100] = np.float16(65504)
    x[130] = np.float16(3000)                                       # one large input among ordinary ones
    x[200] = np.float16(6e-8)                                       # the smallest subnormal among ordinary ones
    for case in ("finite", "inf", "nan"):
        if case == "inf":
            x[300] = np.inf
            x[40] = -np.inf
        if case == "nan":
            x[450] = np.nan
        ref = np.zeros(m, dtype=np.float16)
        oracle.awqo_linear(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(x), ptr(ref), 1)
        got = gemv_gpu(awq, lib, torch, packed, scale, zp, m, k, x)[0]
        print("gemv range", m, k, case, flush=True)
        assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))
        if case == "finite":
            assert not np.any(np.isnan(ref))                        # a large sum may round to an infinity
        else:
            assert np.all(ref.view(np.uint16) == 0x7e00)            # every row sums every block


def test_gemv_unembed_shape_and_argmax(awq, lib, oracle, torch_gpu):
    """config 3: 151936 x 4096 unembedding (scale-group period 32) followed by greedy argmax"""
    torch = torch_gpu
    m, k = 151936, 4096
    rng = np.random.default_rng(3)
    packed, scale, zp = rand_awq(rng, m, k)
    x = rng.standard_normal(k).astype(np.float16)
    ref = np.zeros(m, dtype=np.float16)
    oracle.awqo_linear(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(x), ptr(ref), 1)
    got = gemv_gpu(awq, lib, torch, packed, scale, zp, m, k, x)[0]
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))
    d_l = dev(torch, got)
    ws = torch.zeros(lib.awq_argmax_workspace_bytes(m), dtype=torch.uint8, device="cuda")
    tok = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    awq.check(lib.awq_logits_argmax(d_l.data_ptr(), m, tok.data_ptr(), ws.data_ptr(), stream(torch)))
    torch.cuda.synchronize()
    assert int(tok.item()) == oracle.awqo_argmax(ptr(ref), m)


def test_gemv_one_hot_column_major(awq, lib, torch_gpu):
    torch = torch_gpu
    m, k = 256, 512
    scale = np.ones(m // 128, dtype=np.float16)
    zp = np.zeros(m // 128, dtype=np.float16)
    x = (np.arange(k) % 13 + 1).astype(np.float16)
    for p, q in [(0, 5), (1, 9), (m - 1, 3), (m, 7), (3 * m + 17, 15), (k * m - 1, 1)]:
        packed = np.zeros(m * k // 2, dtype=np.uint8)
        packed[p >> 1] = q << (4 * (p & 1))
        y = gemv_gpu(awq, lib, torch, packed, scale, zp, m, k, x)[0].astype(np.float64)
        expect = np.zeros(m)
        expect[p % m] = q * float(x[p // m])
        assert np.array_equal(y, expect), p


def test_gemv_rejects_bad_shapes(awq, lib, torch_gpu):
    torch = torch_gpu
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    p = buf.data_ptr()
    assert lib.awq_gemv(p, p, p, 100, 512, p, p, p, None) != 0
    assert b"multiple of 128" in lib.awq_last_error()
    assert lib.awq_gemv(p, p, p, 128, 384, p, p, p, None) != 0
    assert lib.awq_linear_repack(p, p, 128, 512, None) != 0
    assert lib.awq_dequant(p, p, p, p, 4, 7, 1, None) != 0


# ----------------------------------------------------------------------------- small operators
@pytest.mark.parametrize("n", [256, 4096])
def test_rmsnorm_bit_exact(awq, lib, oracle, torch_gpu, n):
    torch = torch_gpu
    rng = np.random.default_rng(n)
    for scale_x in [1.0, 30.0, 1e-3]:
        x = (rng.standard_normal(n) * scale_x).astype(np.float16)
        gamma = (1 + 0.02 * rng.standard_normal(n)).astype(np.float16)
        ref = np.zeros(n, dtype=np.float16)
        oracle.awqo_rmsnorm(ptr(x), ptr(gamma), ptr(ref), n, 1e-6)
        d_x, d_g = dev(torch, x), dev(torch, gamma)
        d_o = torch.zeros(n, dtype=torch.float16, device="cuda")
        awq.check(lib.awq_rmsnorm(d_x.data_ptr(), d_g.data_ptr(), d_o.data_ptr(), n, 1e-6, stream(torch)))
        torch.cuda.synchronize()
        assert np.array_equal(d_o.cpu().numpy().view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("n,eps", [(256, 1e-6), (256, 0.0), (768, 1e-6)])
def test_rmsnorm_scale_sweep(awq, lib, oracle, torch_gpu, n, eps):
    """The scale 1/sqrt(mean + eps) over 4000 magnitudes from 1e-4 to 250, an all-zero and a huge vector (the scale is
    then subnormal in binary16), with and without eps and for a length that is no power of two: every output bit
    for bit the oracle's, which pins the divide / square root / divide sequence on the device."""
    torch = torch_gpu
    rng = np.random.default_rng(n + int(eps * 1e7))
    rows = 4000
    mag = np.exp(rng.uniform(np.log(1e-4), np.log(250.0), rows))
    x = (rng.standard_normal((rows + 2, n)) * np.append(mag, [0.0, 1.0])[:, None]).astype(np.float16)
    x[rows + 1] = np.float16(60000.0)
    if eps == 0.0:
        x[rows] = np.float16(1.0)  # 0 * inf: the NaN's sign differs between x86 and the device
    gamma = (1 + 0.02 * rng.standard_normal(n)).astype(np.float16)
    ref = np.zeros_like(x)
    for i in range(rows + 2):
        oracle.awqo_rmsnorm(ptr(x[i]), ptr(gamma), ptr(ref[i]), n, eps)
    d_x, d_g = dev(torch, x), dev(torch, gamma)
    d_o = torch.zeros((rows + 2, n), dtype=torch.float16, device="cuda")
    for i in range(rows + 2):
        awq.check(lib.awq_rmsnorm(d_x.data_ptr() + 2 * n * i, d_g.data_ptr(), d_o.data_ptr() + 2 * n * i, n, eps,
                                  stream(torch)))
    torch.cuda.synchronize()
    assert np.array_equal(d_o.cpu().numpy().view(np.uint16), ref.view(np.uint16))


def test_rope_kv_append_bit_exact(awq, lib, oracle, torch_gpu):
    torch = torch_gpu
    nh, mp = 32, 640
    rng = np.random.default_rng(5)
    cos_t = np.zeros((mp, 64), dtype=np.float16)
    sin_t = np.zeros((mp, 64), dtype=np.float16)
    awq.check(lib.awq_rope_tables_host(ptr(cos_t), ptr(sin_t), mp))
    oc, os_ = np.zeros_like(cos_t), np.zeros_like(sin_t)
    oracle.awqo_rope_tables(ptr(oc), ptr(os_), mp)
    assert np.array_equal(cos_t.view(np.uint16), oc.view(np.uint16)) and np.array_equal(sin_t.view(np.uint16), os_.view(np.uint16))
    H = nh * 128
    d_c, d_s = dev(torch, cos_t), dev(torch, sin_t)
    d_k = torch.zeros(nh * mp * 128, dtype=torch.float16, device="cuda")
    d_v = torch.zeros(nh * mp * 128, dtype=torch.float16, device="cuda")
    kref = np.zeros(nh * mp * 128, dtype=np.float16)
    vref = np.zeros(nh * mp * 128, dtype=np.float16)
    for pos in [0, 1, 512, mp - 1]:
        qkv = rng.standard_normal(3 * H).astype(np.float16)
        q_ref, k_ref, v_ref = qkv[:H].copy(), qkv[H:2 * H].copy(), qkv[2 * H:].copy()
        oracle.awqo_rotary(ptr(q_ref), ptr(oc), ptr(os_), nh, pos)
        oracle.awqo_rotary(ptr(k_ref), ptr(oc), ptr(os_), nh, pos)
        oracle.awqo_kv_append(ptr(kref), ptr(k_ref), nh, mp, pos)
        oracle.awqo_kv_append(ptr(vref), ptr(v_ref), nh, mp, pos)
        d_qkv = dev(torch, qkv)
        d_q = torch.zeros(H, dtype=torch.float16, device="cuda")
        awq.check(lib.awq_rope_kv_append(d_qkv.data_ptr(), d_c.data_ptr(), d_s.data_ptr(), d_q.data_ptr(),
                                         d_k.data_ptr(), d_v.data_ptr(), nh, mp, pos, stream(torch)))
        torch.cuda.synchronize()
        assert np.array_equal(d_q.cpu().numpy().view(np.uint16), q_ref.view(np.uint16)), pos
    assert np.array_equal(d_k.cpu().numpy().view(np.uint16), kref.view(np.uint16))
    assert np.array_equal(d_v.cpu().numpy().view(np.uint16), vref.view(np.uint16))
    assert lib.awq_rope_kv_append(d_qkv.data_ptr(), d_c.data_ptr(), d_s.data_ptr(), d_q.data_ptr(), d_k.data_ptr(),
                                  d_v.data_ptr(), nh, mp, mp, stream(torch)) != 0  # pos out of range


@pytest.mark.parametrize("L", [1, 2, 63, 64, 65, 129, 513, 576, 577, 704, 705, 1500])
def test_decode_attention_bit_exact(awq, lib, oracle, torch_gpu, L):
    torch = torch_gpu
    nh, mp = 32, 2048
    rng = np.random.default_rng(L)
    q = rng.standard_normal(nh * 128).astype(np.float16)
    kc = np.zeros((nh, mp, 128), dtype=np.float16)
    vc = np.zeros((nh, mp, 128), dtype=np.float16)
    kc[:, :L] = rng.standard_normal((nh, L, 128)).astype(np.float16)
    vc[:, :L] = rng.standard_normal((nh, L, 128)).astype(np.float16)
    # positions past L hold garbage that must not be read into the result
    kc[:, L:L + 3] = np.float16(1000.0)
    vc[:, L:L + 3] = np.float16("inf")
    ref = np.zeros(nh * 128, dtype=np.float16)
    oracle.awqo_attention(ptr(q), ptr(kc), ptr(vc), ptr(ref), nh, mp, L, None)
    d_q, d_k, d_v = dev(torch, q), dev(torch, kc), dev(torch, vc)
    d_o = torch.zeros(nh * 128, dtype=torch.float16, device="cuda")
    ws = torch.zeros(lib.awq_attention_workspace_bytes(nh, mp), dtype=torch.uint8, device="cuda")
    print("attention L", L, flush=True)
    awq.check(lib.awq_decode_attention(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), d_o.data_ptr(), nh, mp, L,
                                       ws.data_ptr(), stream(torch)))
    torch.cuda.synchronize()
    assert np.array_equal(d_o.cpu().numpy().view(np.uint16), ref.view(np.uint16))
    if L == 1:
        assert np.array_equal(d_o.cpu().numpy().reshape(nh, 128).view(np.uint16), vc[:, 0].view(np.uint16))
    assert lib.awq_decode_attention(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), d_o.data_ptr(), nh, mp, mp + 1,
                                    ws.data_ptr(), stream(torch)) != 0


@pytest.mark.parametrize("L", [577, 704, 705, 1000, 1024, 1025, 2048, 2049, 4097, 9001, 20000])
def test_decode_attention_long_sequences_bit_exact(awq, lib, oracle, torch_gpu, L):
    """beyond 704 positions the launches are cut along the sequence (32 parts per head, some of them
    empty while the sequence has fewer than 32 chunks; two launches up to 1024 positions, three up to 2048,
    four beyond);
    the summation orders are those of the short
    path, so the oracle's bits must come out"""
    torch = torch_gpu
    nh, mp = 4, 20480
    rng = np.random.default_rng(L)
    q = rng.standard_normal(nh * 128).astype(np.float16)
    kc = np.zeros((nh, mp, 128), dtype=np.float16)
    vc = np.zeros((nh, mp, 128), dtype=np.float16)
    kc[:, :L] = (0.3 * rng.standard_normal((nh, L, 128))).astype(np.float16)
    vc[:, :L] = rng.standard_normal((nh, L, 128)).astype(np.float16)
    kc[:, L:L + 3] = np.float16(1000.0)
    vc[:, L:L + 3] = np.float16("inf")
    ref = np.zeros(nh * 128, dtype=np.float16)
    oracle.awqo_attention(ptr(q), ptr(kc), ptr(vc), ptr(ref), nh, mp, L, None)
    d_q, d_k, d_v = dev(torch, q), dev(torch, kc), dev(torch, vc)
    d_o = torch.zeros(nh * 128, dtype=torch.float16, device="cuda")
    ws = torch.zeros(lib.awq_attention_workspace_bytes(nh, mp), dtype=torch.uint8, device="cuda")
    print("attention, long sequence, L", L, flush=True)
    for _ in range(2):   # the workspace holds the previous call's values the second time
        awq.check(lib.awq_decode_attention(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), d_o.data_ptr(), nh, mp, L,
                                           ws.data_ptr(), stream(torch)))
        torch.cuda.synchronize()
        assert np.array_equal(d_o.cpu().numpy().view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("pos0,M,first_layer", [(0, 1, 1), (0, 37, 1), (0, 130, 0), (70, 150, 0), (2040, 40, 0), (5, 64, 1)])
def test_prefill_attention_matches_the_one_query_path(awq, lib, oracle, torch_gpu, pos0, M, first_layer):
    """attention of M prompt positions at once on the matrix cores against the oracle's one-query
    attention with each token's own attended length; 1e-2 of the largest output magnitude"""
    torch = torch_gpu
    nh, mp = 4, 2112
    rng = np.random.default_rng(pos0 * 1000 + M)
    n_pos = pos0 + M
    q = rng.standard_normal((M, nh * 128)).astype(np.float16)
    kc = np.zeros((nh, mp, 128), dtype=np.float16)
    vc = np.zeros((nh, mp, 128), dtype=np.float16)
    kc[:, :n_pos] = (0.5 * rng.standard_normal((nh, n_pos, 128))).astype(np.float16)
    vc[:, :n_pos] = rng.standard_normal((nh, n_pos, 128)).astype(np.float16)
    ref = np.zeros((M, nh * 128), dtype=np.float16)
    for t in range(M):
        p = pos0 + t
        L = max(p, 1) if first_layer else p + 1
        row = np.zeros(nh * 128, dtype=np.float16)
        oracle.awqo_attention(ptr(np.ascontiguousarray(q[t])), ptr(kc), ptr(vc), ptr(row), nh, mp, L, None)
        ref[t] = row
    d_q, d_k, d_v = dev(torch, q), dev(torch, kc), dev(torch, vc)
    d_o = torch.full((M, nh * 128), float("nan"), dtype=torch.float16, device="cuda")
    print("prefill attention", pos0, M, first_layer, flush=True)
    awq.check(lib.awq_prefill_attention(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), d_o.data_ptr(), nh, mp, pos0, M,
                                        first_layer, stream(torch)))
    torch.cuda.synchronize()
    got = d_o.cpu().numpy().astype(np.float64)
    want = ref.astype(np.float64)
    assert np.all(np.isfinite(got))
    assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max()
    assert lib.awq_prefill_attention(d_q.data_ptr(), d_k.data_ptr(), d_v.data_ptr(), d_o.data_ptr(), nh, mp, mp - 1, 2,
                                     0, stream(torch)) != 0     # runs past max_pos


def test_gelu_all_fp16_values_and_residual(awq, lib, oracle, torch_gpu):
    torch = torch_gpu
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    allh = allh[np.isfinite(allh)].copy()
    ref = allh.copy()
    oracle.awqo_gelu(ptr(ref), ref.size)
    d = dev(torch, allh)
    awq.check(lib.awq_gelu(d.data_ptr(), allh.size, stream(torch)))
    torch.cuda.synchronize()
    assert np.array_equal(d.cpu().numpy().view(np.uint16), ref.view(np.uint16))
    rng = np.random.default_rng(9)
    a = (rng.standard_normal(4096) * 4).astype(np.float16)
    b = (rng.standard_normal(4096) * 4).astype(np.float16)
    ref = np.zeros_like(a)
    oracle.awqo_residual(ptr(a), ptr(b), ptr(ref), a.size)
    d_a, d_b = dev(torch, a), dev(torch, b)
    awq.check(lib.awq_residual_add(d_a.data_ptr(), d_b.data_ptr(), d_a.data_ptr(), a.size, stream(torch)))
    torch.cuda.synchronize()
    assert np.array_equal(d_a.cpu().numpy().view(np.uint16), ref.view(np.uint16))


def test_argmax_rules(awq, lib, oracle, torch_gpu):
    torch = torch_gpu
    n = 151936
    rng = np.random.default_rng(11)
    ws = torch.zeros(lib.awq_argmax_workspace_bytes(n), dtype=torch.uint8, device="cuda")
    tok = torch.zeros(1, dtype=torch.int32, device="cuda")

    def run(x):
        d = dev(torch, x)
        awq.check(lib.awq_logits_argmax(d.data_ptr(), x.size, tok.data_ptr(), ws.data_ptr(), stream(torch)))
        torch.cuda.synchronize()
        return int(tok.item())

    cases = []
    x = np.zeros(n, dtype=np.float16); cases.append(x.copy())
    x[[10, 70000, n - 1]] = 3.5; cases.append(x.copy())
    x[90000] = np.float16("nan"); cases.append(x.copy())
    x[0] = np.float16("nan"); cases.append(x.copy())
    x[:] = -np.inf; x[77] = -65504.0; cases.append(x.copy())
    x[:] = 0.0; x[5] = -0.0; cases.append(x.copy())
    x[:] = np.float16("nan"); cases.append(x.copy())
    for _ in range(4):
        cases.append((rng.standard_normal(n) * 5).astype(np.float16))  # plenty of exact FP16 ties near the top
    cases.append(rng.integers(-3, 4, size=n).astype(np.float16))
    cases.append(rng.standard_normal(1000).astype(np.float16))
    for c in cases:
        assert run(c) == oracle.awqo_argmax(ptr(c), c.size)


def test_embed_gather_bit_exact(awq, lib, oracle, torch_gpu):
    torch = torch_gpu
    H, V = 512, 4096
    rng = np.random.default_rng(13)
    packed, scale, zp = rand_awq(rng, H, V)
    d_p, d_s, d_z = dev(torch, packed), dev(torch, scale), dev(torch, zp)
    d_o = torch.zeros(H, dtype=torch.float16, device="cuda")
    ref = np.zeros(H, dtype=np.float16)
    for tok in [0, 1, 127, 128, 1000, 4095]:
        oracle.awqo_embed(ptr(packed), ptr(scale), ptr(zp), H, V, tok, ptr(ref))
        awq.check(lib.awq_embed_gather(d_p.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), H, V, tok, d_o.data_ptr(),
                                       stream(torch)))
        torch.cuda.synchronize()
        assert np.array_equal(d_o.cpu().numpy().view(np.uint16), ref.view(np.uint16)), tok
    assert lib.awq_embed_gather(d_p.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), H, V, V, d_o.data_ptr(), None) != 0


# ----------------------------------------------------------------------------- fused linear launches
def fused_setup(awq, lib, torch, rng, m, k, zp_int=True):
    packed, scale, zp = rand_awq(rng, m, k, zp_int=zp_int)
    d_in = dev(torch, packed)
    d_w = torch.zeros(m * k // 2, dtype=torch.uint8, device="cuda")
    awq.check(lib.awq_linear_repack(d_in.data_ptr(), d_w.data_ptr(), m, k, stream(torch)))
    keep = dict(d_w=d_w, d_s=dev(torch, scale), d_z=dev(torch, zp),
                ws=torch.zeros(lib.awq_gemv_workspace_bytes(m, k), dtype=torch.uint8, device="cuda"))
    a = awq.AwqLinearArgs()
    a.repacked, a.scale, a.zp = keep["d_w"].data_ptr(), keep["d_s"].data_ptr(), keep["d_z"].data_ptr()
    a.m, a.k, a.workspace = m, k, keep["ws"].data_ptr()
    return packed, scale, zp, a, keep


# the last two: more than 1024 row groups, so a workgroup walks several of them and runs the epilogues of all its
# passes at the end (one scale group per 16 rows, and a scale group that depends on the input index)
@pytest.mark.parametrize("m,k", [(256, 512), (12288, 4096), (4096, 12288), (20480, 1024), (128 * 147, 512)])
def test_gemv_fused_norm_gelu_residual(awq, lib, oracle, torch_gpu, m, k):
    torch = torch_gpu
    rng = np.random.default_rng(m + 3 * k)
    packed, scale, zp, a, keep = fused_setup(awq, lib, torch, rng, m, k)
    hidden = (rng.standard_normal(k) * 2).astype(np.float16)
    gamma = (1 + 0.02 * rng.standard_normal(k)).astype(np.float16)
    res = rng.standard_normal(m).astype(np.float16)
    normed = np.zeros(k, dtype=np.float16)
    oracle.awqo_rmsnorm(ptr(hidden), ptr(gamma), ptr(normed), k, 1e-6)
    lin = np.zeros(m, dtype=np.float16)
    oracle.awqo_linear(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(normed), ptr(lin), 1)
    d_h, d_g, d_r = dev(torch, hidden), dev(torch, gamma), dev(torch, res)
    d_y = torch.zeros(m, dtype=torch.float16, device="cuda")
    a.x, a.y, a.gamma, a.eps = d_h.data_ptr(), d_y.data_ptr(), d_g.data_ptr(), 1e-6
    # RMSNorm prologue, plain store
    a.prologue, a.epilogue = awq.PRO_RMSNORM, awq.EPI_STORE
    awq.check(lib.awq_gemv_fused(ctypes.byref(a), stream(torch)))
    torch.cuda.synchronize()
    assert np.array_equal(d_y.cpu().numpy().view(np.uint16), lin.view(np.uint16))
    # RMSNorm prologue + GeLU epilogue (the W1 launch)
    a.epilogue = awq.EPI_GELU
    awq.check(lib.awq_gemv_fused(ctypes.byref(a), stream(torch)))
    torch.cuda.synchronize()
    g = lin.copy()
    oracle.awqo_gelu(ptr(g), m)
    assert np.array_equal(d_y.cpu().numpy().view(np.uint16), g.view(np.uint16))
    # residual epilogue in place (the Wo / W2 launches)
    a.prologue, a.epilogue = awq.PRO_NONE, awq.EPI_RESIDUAL
    d_n = dev(torch, normed)
    a.x, a.y, a.residual = d_n.data_ptr(), d_r.data_ptr(), d_r.data_ptr()
    awq.check(lib.awq_gemv_fused(ctypes.byref(a), stream(torch)))
    torch.cuda.synchronize()
    rr = np.zeros(m, dtype=np.float16)
    oracle.awqo_residual(ptr(res), ptr(lin), ptr(rr), m)
    assert np.array_equal(d_r.cpu().numpy().view(np.uint16), rr.view(np.uint16))


@pytest.mark.parametrize("H,pos", [(512, 0), (512, 5), (4096, 512)])
def test_gemv_fused_qkv_rope_kv_append(awq, lib, oracle, torch_gpu, H, pos):
    """config 2's first launch: RMSNorm + Wqkv + split + rotary + KV append"""
    torch = torch_gpu
    m, k, nh, mp = 3 * H, H, H // 128, 640
    rng = np.random.default_rng(H + pos)
    packed, scale, zp, a, keep = fused_setup(awq, lib, torch, rng, m, k)
    hidden = rng.standard_normal(k).astype(np.float16)
    gamma = (1 + 0.02 * rng.standard_normal(k)).astype(np.float16)
    cos_t, sin_t = np.zeros((mp, 64), np.float16), np.zeros((mp, 64), np.float16)
    oracle.awqo_rope_tables(ptr(cos_t), ptr(sin_t), mp)
    normed = np.zeros(k, dtype=np.float16)
    oracle.awqo_rmsnorm(ptr(hidden), ptr(gamma), ptr(normed), k, 1e-6)
    qkv = np.zeros(m, dtype=np.float16)
    oracle.awqo_linear(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(normed), ptr(qkv), 1)
    q_ref, k_ref, v_ref = qkv[:H].copy(), qkv[H:2 * H].copy(), qkv[2 * H:].copy()
    oracle.awqo_rotary(ptr(q_ref), ptr(cos_t), ptr(sin_t), nh, pos)
    oracle.awqo_rotary(ptr(k_ref), ptr(cos_t), ptr(sin_t), nh, pos)
    kc_ref = rng.standard_normal(nh * mp * 128).astype(np.float16)
    vc_ref = rng.standard_normal(nh * mp * 128).astype(np.float16)
    d_kc, d_vc = dev(torch, kc_ref), dev(torch, vc_ref)
    oracle.awqo_kv_append(ptr(kc_ref), ptr(k_ref), nh, mp, pos)
    oracle.awqo_kv_append(ptr(vc_ref), ptr(v_ref), nh, mp, pos)
    d_h, d_g, d_c, d_s = dev(torch, hidden), dev(torch, gamma), dev(torch, cos_t), dev(torch, sin_t)
    d_q = torch.zeros(H, dtype=torch.float16, device="cuda")
    a.x, a.y, a.gamma, a.eps = d_h.data_ptr(), d_q.data_ptr(), d_g.data_ptr(), 1e-6
    a.prologue, a.epilogue = awq.PRO_RMSNORM, awq.EPI_QKV_ROPE
    a.cos_t, a.sin_t, a.k_cache, a.v_cache = d_c.data_ptr(), d_s.data_ptr(), d_kc.data_ptr(), d_vc.data_ptr()
    a.hidden, a.max_pos, a.pos = H, mp, pos
    awq.check(lib.awq_gemv_fused(ctypes.byref(a), stream(torch)))
    torch.cuda.synchronize()
    assert np.array_equal(d_q.cpu().numpy().view(np.uint16), q_ref.view(np.uint16))
    assert np.array_equal(d_kc.cpu().numpy().view(np.uint16), kc_ref.view(np.uint16))
    assert np.array_equal(d_vc.cpu().numpy().view(np.uint16), vc_ref.view(np.uint16))
    a.pos = mp
    assert lib.awq_gemv_fused(ctypes.byref(a), stream(torch)) != 0


@pytest.mark.parametrize("m,k", [(128 * 37, 512), (151936, 4096)])
def test_gemv_fused_norm_unembed_argmax(awq, lib, oracle, torch_gpu, m, k):
    """config 3: final RMSNorm + unembedding + greedy argmax in one launch"""
    torch = torch_gpu
    rng = np.random.default_rng(m)
    packed, scale, zp, a, keep = fused_setup(awq, lib, torch, rng, m, k)
    gamma = (1 + 0.02 * rng.standard_normal(k)).astype(np.float16)
    d_g = dev(torch, gamma)
    tok = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    d_y = torch.zeros(m, dtype=torch.float16, device="cuda")
    for trial in range(3):
        hidden = rng.standard_normal(k).astype(np.float16)
        normed = np.zeros(k, dtype=np.float16)
        oracle.awqo_rmsnorm(ptr(hidden), ptr(gamma), ptr(normed), k, 1e-6)
        logits = np.zeros(m, dtype=np.float16)
        oracle.awqo_linear(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(normed), ptr(logits), 1)
        d_h = dev(torch, hidden)
        a.x, a.y, a.gamma, a.eps, a.out_token = d_h.data_ptr(), d_y.data_ptr(), d_g.data_ptr(), 1e-6, tok.data_ptr()
        a.prologue, a.epilogue = awq.PRO_RMSNORM, awq.EPI_ARGMAX
        awq.check(lib.awq_gemv_fused(ctypes.byref(a), stream(torch)))
        torch.cuda.synchronize()
        assert np.array_equal(d_y.cpu().numpy().view(np.uint16), logits.view(np.uint16))
        assert int(tok.item()) == oracle.awqo_argmax(ptr(logits), m)
    assert int(keep["ws"].to(torch.int32).abs().sum().item()) == 0  # sampler workspace left zeroed


# ----------------------------------------------------------------------------- Wqkv + attention as one launch
@pytest.mark.parametrize("pos,L", [(0, 1), (1, 1), (2, 2), (2, 3), (5, 5), (63, 64), (70, 71), (300, 301), (640, 640),
                                   (703, 704), (704, 705), (959, 960), (960, 961), (1023, 1023), (1023, 1024),
                                   (1024, 1025), (1500, 1501), (1984, 1985), (2047, 2048), (2048, 2049), (3000, 2950),
                                   (3007, 3008), (3071, 3072), (3072, 3073), (4031, 4032), (4095, 4096)])
def test_fused_qkv_attention_launch_against_the_two_launches_and_the_oracle(awq, lib, oracle, torch_gpu, pos, L):
    """awq_qkv_attention: RMSNorm + Wqkv + rotary + KV append and the attention over the cache in one launch whose
    eight workgroups per head hand partial scores to each other through the L2 of their die.  Q, the caches and
    the context must be those of awq_gemv_fused + awq_decode_attention and of the oracle, bit for bit, on two
    calls in a row (the tags change; the second call finds the first one's words in the exchange buffer)."""
    torch = torch_gpu
    H = 4096
    m, k, nh, mp = 3 * H, H, H // 128, (2112 if pos < 2112 else 4160)
    if not lib.awq_qkv_attention_supported(H, nh, stream(torch)):
        pytest.skip("this device cannot run the fused launch")
    rng = np.random.default_rng(pos * 1000 + L)
    packed, scale, zp, a, keep = fused_setup(awq, lib, torch, rng, m, k)
    hidden = rng.standard_normal(k).astype(np.float16)
    gamma = (1 + 0.02 * rng.standard_normal(k)).astype(np.float16)
    cos_t, sin_t = np.zeros((mp, 64), np.float16), np.zeros((mp, 64), np.float16)
    oracle.awqo_rope_tables(ptr(cos_t), ptr(sin_t), mp)
    kc = (rng.standard_normal(nh * mp * 128) * 0.3).astype(np.float16)
    vc = rng.standard_normal(nh * mp * 128).astype(np.float16)
    d_h, d_g, d_c, d_s = dev(torch, hidden), dev(torch, gamma), dev(torch, cos_t), dev(torch, sin_t)
    # the oracle
    normed = np.zeros(k, dtype=np.float16)
    oracle.awqo_rmsnorm(ptr(hidden), ptr(gamma), ptr(normed), k, 1e-6)
    qkv = np.zeros(m, dtype=np.float16)
    oracle.awqo_linear(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(normed), ptr(qkv), 1)
    q_ref, k_ref, v_ref = qkv[:H].copy(), qkv[H:2 * H].copy(), qkv[2 * H:].copy()
    oracle.awqo_rotary(ptr(q_ref), ptr(cos_t), ptr(sin_t), nh, pos)
    oracle.awqo_rotary(ptr(k_ref), ptr(cos_t), ptr(sin_t), nh, pos)
    kc_ref, vc_ref = kc.copy(), vc.copy()
    oracle.awqo_kv_append(ptr(kc_ref), ptr(k_ref), nh, mp, pos)
    oracle.awqo_kv_append(ptr(vc_ref), ptr(v_ref), nh, mp, pos)
    ctx_ref = np.zeros(H, dtype=np.float16)
    oracle.awqo_attention(ptr(q_ref), ptr(kc_ref), ptr(vc_ref), ptr(ctx_ref), nh, mp, L, None)
    # two launches
    d_kc, d_vc = dev(torch, kc), dev(torch, vc)
    d_q = torch.zeros(H, dtype=torch.float16, device="cuda")
    d_o = torch.zeros(H, dtype=torch.float16, device="cuda")
    a.x, a.y, a.gamma, a.eps = d_h.data_ptr(), d_q.data_ptr(), d_g.data_ptr(), 1e-6
    a.prologue, a.epilogue = awq.PRO_RMSNORM, awq.EPI_QKV_ROPE
    a.cos_t, a.sin_t, a.k_cache, a.v_cache = d_c.data_ptr(), d_s.data_ptr(), d_kc.data_ptr(), d_vc.data_ptr()
    a.hidden, a.max_pos, a.pos = H, mp, pos
    awq.check(lib.awq_gemv_fused(ctypes.byref(a), stream(torch)))
    ws = torch.zeros(lib.awq_attention_workspace_bytes(nh, mp), dtype=torch.uint8, device="cuda")
    awq.check(lib.awq_decode_attention(d_q.data_ptr(), d_kc.data_ptr(), d_vc.data_ptr(), d_o.data_ptr(), nh, mp, L,
                                       ws.data_ptr(), stream(torch)))
    torch.cuda.synchronize()
    assert np.array_equal(d_o.cpu().numpy().view(np.uint16), ctx_ref.view(np.uint16))
    # one launch
    f_kc, f_vc = dev(torch, kc), dev(torch, vc)
    f_q = torch.zeros(H, dtype=torch.float16, device="cuda")
    f_o = torch.zeros(H, dtype=torch.float16, device="cuda")
    fws = torch.zeros(lib.awq_qkv_attention_workspace_bytes(nh), dtype=torch.uint8, device="cuda")
    # the caches a second time in the launch's own order, [head][8][pp][16]: the rows before pos are copied, the
    # launch appends row pos itself
    pp = 2048 if pos < 2048 else 4096
    assert lib.awq_kv_parts_bytes(nh, pp) == nh * 128 * pp * 2
    f_kp = torch.full((nh * 8 * pp * 16,), 7.0, dtype=torch.float16, device="cuda")
    f_vp = torch.full((nh * 8 * pp * 16,), 7.0, dtype=torch.float16, device="cuda")
    awq.check(lib.awq_kv_cache_to_parts(f_kc.data_ptr(), f_vc.data_ptr(), mp, nh, f_kp.data_ptr(), f_vp.data_ptr(), pp, 0,
                                        pos, stream(torch)))
    print("fused launch pos", pos, "L", L, flush=True)
    args = [keep["d_w"].data_ptr(), keep["d_s"].data_ptr(), keep["d_z"].data_ptr(), d_h.data_ptr(), d_g.data_ptr(), 1e-6,
            d_c.data_ptr(), d_s.data_ptr(), f_kc.data_ptr(), f_vc.data_ptr(), mp, f_kp.data_ptr(), f_vp.data_ptr(), pp, nh,
            pos, L, f_q.data_ptr(), f_o.data_ptr(), fws.data_ptr(), 3, stream(torch)]
    for call in (1, 2):
        f_o.zero_()
        args[20] = call
        awq.check(lib.awq_qkv_attention(*args))
        awq.check(lib.awq_qkv_attention_status(fws.data_ptr(), stream(torch)))
        assert np.array_equal(f_q.cpu().numpy().view(np.uint16), q_ref.view(np.uint16))
        assert np.array_equal(f_kc.cpu().numpy().view(np.uint16), kc_ref.view(np.uint16))
        assert np.array_equal(f_vc.cpu().numpy().view(np.uint16), vc_ref.view(np.uint16))
        assert np.array_equal(f_o.cpu().numpy().view(np.uint16), ctx_ref.view(np.uint16))
        assert np.array_equal(f_o.cpu().numpy().view(np.uint16), d_o.cpu().numpy().view(np.uint16))
        # the second copy: rows 0..pos of the caches, dimension 16 p + d of head h at [h][p][position][d]; nothing else written
        for parts, ref in ((f_kp, kc_ref), (f_vp, vc_ref)):
            got = parts.cpu().numpy().view(np.uint16).reshape(nh, 8, pp, 16)
            want = ref.view(np.uint16).reshape(nh, mp, 8, 16)[:, :pos + 1].transpose(0, 2, 1, 3)
            assert np.array_equal(got[:, :, :pos + 1], want)
            assert (got[:, :, pos + 1:] == np.float16(7.0).view(np.uint16)).all()
    # arguments the launch is not built for are refused before anything runs
    args[20] = 3
    for idx, bad in ((14, 16), (15, mp), (16, pos + 2), (20, 0), (13, L - 1)):
        wrong = list(args)
        wrong[idx] = bad
        assert lib.awq_qkv_attention(*wrong) != 0
    assert lib.awq_kv_cache_to_parts(f_kc.data_ptr(), f_vc.data_ptr(), mp, nh, f_kp.data_ptr(), f_vp.data_ptr(), pp, pp - 1,
                                     2, stream(torch)) != 0
    # the copy by itself: no rows is no work; rows from the middle land where they belong and nowhere else
    if pos >= 70:
        t_kp = torch.full_like(f_kp, 3.0)
        t_vp = torch.full_like(f_vp, 3.0)
        awq.check(lib.awq_kv_cache_to_parts(f_kc.data_ptr(), f_vc.data_ptr(), mp, nh, t_kp.data_ptr(), t_vp.data_ptr(), pp, 5, 0,
                                            stream(torch)))
        assert (t_kp == 3.0).all() and (t_vp == 3.0).all()
        awq.check(lib.awq_kv_cache_to_parts(f_kc.data_ptr(), f_vc.data_ptr(), mp, nh, t_kp.data_ptr(), t_vp.data_ptr(), pp, 5, 60,
                                            stream(torch)))
        for parts, ref in ((t_kp, kc_ref), (t_vp, vc_ref)):
            got = parts.cpu().numpy().view(np.uint16).reshape(nh, 8, pp, 16)
            want = ref.view(np.uint16).reshape(nh, mp, 8, 16)[:, 5:65].transpose(0, 2, 1, 3)
            assert np.array_equal(got[:, :, 5:65], want)
            three = np.float16(3.0).view(np.uint16)
            assert (got[:, :, :5] == three).all() and (got[:, :, 65:] == three).all()


# ----------------------------------------------------------------------------- W4A16 GEMM on the matrix cores
@pytest.mark.parametrize("m,k,M,zp_int", [(256, 512, 3, True), (256, 512, 17, False), (384, 1536, 130, True),
                                          (12288, 4096, 16, True), (12288, 4096, 200, True), (4096, 12288, 64, False),
                                          (4096, 12288, 128, True), (12288, 4096, 1030, True),
                                          (4096, 4096, 1024, True), (4096, 12288, 1024, True),
                                          (4096, 12288, 640, True), (384, 6144, 8500, False),
                                          # config 5's own points: the 2048-token prefill product and the
                                          # decode-batch sweep M = 1, 4, 16, 64 on the w1 and w2 shapes
                                          (12288, 4096, 2048, True), (4096, 12288, 2048, True),
                                          (12288, 4096, 1, True), (4096, 12288, 1, True),
                                          (12288, 4096, 4, True), (4096, 12288, 4, True),
                                          (4096, 12288, 16, True), (12288, 4096, 64, True),
                                          # 5..16 tokens: several row groups per workgroup (three, with a last
                                          # workgroup of two; two; one), k of 128, 256 and 384 blocks
                                          (12288, 4096, 5, False), (16384, 4096, 11, True), (4096, 8192, 9, False),
                                          (8192, 8192, 13, True), (4096, 12288, 7, True), (4096, 4096, 16, False),
                                          (2048, 16384, 10, True), (4096, 4096, 2, True), (1024, 4096, 3, False),
                                          # 17..64 tokens on 4096 rows, the token tile shared through LDS: two
                                          # and four 16-token tiles, k of 16 and of 8 steps
                                          (4096, 4096, 17, True), (4096, 4096, 32, False), (4096, 4096, 33, True),
                                          (4096, 4096, 64, False), (4096, 2048, 20, True), (4096, 2048, 49, False),
                                          (4096, 4096, 130, True), (4096, 4096, 192, False), (4096, 2048, 150, True),
                                          (12288, 4096, 33, True), (8192, 4096, 49, False),
                                          (12288, 4096, 20, False), (12288, 2048, 40, True), (10240, 2048, 31, False),
                                          # ... and 64 tokens after the other: two slabs, a ragged third, four
                                          (12288, 4096, 65, True), (12288, 4096, 128, False), (12288, 2048, 150, True),
                                          (12288, 4096, 256, True),
                                          # ... with k cut over four workgroups and a second launch
                                          (4096, 12288, 130, False), (4096, 12288, 192, True), (4096, 12288, 320, True)])
def test_gemm_matches_fp32_accumulate_reference(awq, lib, oracle, torch_gpu, m, k, M, zp_int):
    """config 5: dequant-on-load MFMA product; 1e-2 relative against the sequential FP32-accumulate
    reference, and the weights it multiplies are the bit-exact dequantised ones (one-hot check below).
    The shapes cover every workgroup shape: few tokens (3), k split (17, 64, 128, 130 tokens; k also cut
    over workgroups for 4096 x 12288 x 128), rows split with 64 tokens per workgroup (12288 x 4096 x 200,
    4096 x 4096 x 1024), a tile per workgroup (1030 tokens), and work cut evenly with handed-over sums:
    two aligned pieces per tile (4096 x 12288 x 1024 and x 640) and 256 unequal ranges (384 x 6144 x 8500)"""
    torch = torch_gpu
    rng = np.random.default_rng(m + k + M)
    packed, scale, zp = rand_awq(rng, m, k, zp_int=zp_int)
    x = rng.standard_normal((M, k)).astype(np.float16)
    Mo = min(M, 24)  # the oracle is slow on the large shapes: check a subset of tokens there
    sel = np.sort(rng.choice(M, size=Mo, replace=False))
    ref = np.zeros((Mo, m), dtype=np.float16)
    xs = np.ascontiguousarray(x[sel])
    # the reference arithmetic: binary16-dequantised weights (Inference.cu:102-104), binary32 accumulation
    oracle.awqo_linear_seq(ptr(packed), ptr(scale), ptr(zp), m, k, ptr(xs), ptr(ref), Mo)
    d_in = dev(torch, packed)
    d_w = torch.zeros(m * k // 2, dtype=torch.uint8, device="cuda")
    awq.check(lib.awq_linear_repack(d_in.data_ptr(), d_w.data_ptr(), m, k, stream(torch)))
    d_s, d_z, d_x = dev(torch, scale), dev(torch, zp), dev(torch, x)
    d_y = torch.full((M, m), float("nan"), dtype=torch.float16, device="cuda")
    print("gemm", m, k, M, flush=True)
    awq.check(lib.awq_gemm(d_w.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), m, k, d_x.data_ptr(), d_y.data_ptr(), M,
                           1 if zp_int else 0, None, stream(torch)))
    torch.cuda.synchronize()
    # with room for partial sums the product may cut k over several workgroups: same tolerance, and
    # nothing changes where it does not (workspace size 0)
    wsb = lib.awq_gemm_workspace_bytes(m, k, M)
    d_ws = torch.zeros(max(wsb, 16), dtype=torch.uint8, device="cuda")
    d_y2 = torch.full((M, m), float("nan"), dtype=torch.float16, device="cuda")
    awq.check(lib.awq_gemm(d_w.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), m, k, d_x.data_ptr(), d_y2.data_ptr(), M,
                           1 if zp_int else 0, d_ws.data_ptr(), stream(torch)))
    torch.cuda.synchronize()
    got2 = d_y2.cpu().numpy()[sel].astype(np.float64)
    if wsb == 0:
        assert np.array_equal(d_y2.cpu().numpy().view(np.uint16), d_y.cpu().numpy().view(np.uint16))
    else:
        # the header (status word, hand-over counters) is zero again, and a second product on the same
        # workspace gives the same bits: partial sums are added in a fixed order
        assert int(d_ws[:4096].to(torch.int32).sum().item()) == 0
        d_y3 = torch.full((M, m), float("nan"), dtype=torch.float16, device="cuda")
        awq.check(lib.awq_gemm(d_w.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), m, k, d_x.data_ptr(), d_y3.data_ptr(),
                               M, 1 if zp_int else 0, d_ws.data_ptr(), stream(torch)))
        torch.cuda.synchronize()
        assert np.array_equal(d_y3.cpu().numpy().view(np.uint16), d_y2.cpu().numpy().view(np.uint16))
        assert int(d_ws[:4096].to(torch.int32).sum().item()) == 0
    got = d_y.cpu().numpy()[sel].astype(np.float64)
    want = ref.astype(np.float64)
    # 1e-2 relative; outputs smaller than the root mean square of all outputs are measured against that
    # (a sum of 512..12288 terms that cancels to nearly nothing has no relative accuracy to speak of)
    denom = np.maximum(np.abs(want), np.sqrt(np.mean(want * want)))
    assert np.all(np.isfinite(got))
    assert np.all(np.abs(got - want) <= 1e-2 * denom)
    assert np.all(np.isfinite(got2)) and np.all(np.abs(got2 - want) <= 1e-2 * denom)
    # much tighter in practice: both sides accumulate in FP32.  The kernels of up to 16 tokens round every
    # weight twice as Inference.cu:102-104 does and differ from the reference only in the order of the sum;
    # the many-token kernel applies the scale to the sum instead of to every weight (one binary16 rounding
    # fewer per weight).  99% of the outputs within two binary16 roundings.
    p99a, p99b = np.percentile(np.abs(got - want) / denom, 99), np.percentile(np.abs(got2 - want) / denom, 99)
    print("99th percentile of the relative error: %.3g %.3g (2^-10 = %.3g)" % (p99a, p99b, 2.0 ** -10), flush=True)
    assert p99a <= 2.0 ** -10 and p99b <= 2.0 ** -10


def _random_gemm_shapes(n, seed):
    """(m, k, M): multiples of 128 / 512 whose scale group does not depend on the input index"""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        a, r = int(rng.integers(1, 25)), int(rng.choice([1, 2, 3, 4]))
        mg, kg = (a * r, a) if rng.random() < 0.5 else (a, a * r)
        kg = max(4, kg - kg % 4)            # k a multiple of 512
        if not (mg % kg == 0 or kg % mg == 0) or mg > 96 or kg > 96:
            continue
        if not any(kg % g == 0 and kg // g <= 16 for g in (8, 4, 2, 1)):
            continue                        # the weight stream's lane groups (shared with the decode kernel)
        M = int(rng.choice([rng.integers(5, 130), rng.integers(130, 700), rng.integers(700, 2600)]))
        out.append((128 * mg, 128 * kg, M))
    return out


@pytest.mark.parametrize("m,k,M", _random_gemm_shapes(24, 20240607))
def test_gemm_random_shapes_match_torch_fp32(awq, lib, torch_gpu, m, k, M):
    """every workgroup shape the planner can pick, on random matrix shapes and token counts, against an
    FP32 product of the bit-exactly dequantised weights (awq_dequant, itself pinned against the oracle):
    1e-2 relative as above, with and without a workspace"""
    torch = torch_gpu
    rng = np.random.default_rng(m * 31 + k * 7 + M)
    zp_int = bool(rng.integers(0, 2))
    packed, scale, zp = rand_awq(rng, m, k, zp_int=zp_int)
    d_in, d_s, d_z = dev(torch, packed), dev(torch, scale), dev(torch, zp)
    d_dq = torch.zeros(m * k, dtype=torch.float16, device="cuda")
    awq.check(lib.awq_dequant(d_in.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), d_dq.data_ptr(), m, k, m // 128,
                              stream(torch)))
    d_w = torch.zeros(m * k // 2, dtype=torch.uint8, device="cuda")
    awq.check(lib.awq_linear_repack(d_in.data_ptr(), d_w.data_ptr(), m, k, stream(torch)))
    d_x = torch.from_numpy(rng.standard_normal((M, k)).astype(np.float16)).cuda()
    # the reference reads the row-major dequantised buffer column-major: W(i, j) = dq[i + j m]
    want = (d_x.float() @ d_dq.view(k, m).float()).double().cpu().numpy()
    denom = np.maximum(np.abs(want), np.sqrt(np.mean(want * want)))
    for use_ws in (False, True):
        wsb = lib.awq_gemm_workspace_bytes(m, k, M) if use_ws else 0
        d_ws = torch.zeros(max(wsb, 16), dtype=torch.uint8, device="cuda")
        d_y = torch.full((M, m), float("nan"), dtype=torch.float16, device="cuda")
        print("gemm", m, k, M, "workspace", wsb, flush=True)
        awq.check(lib.awq_gemm(d_w.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), m, k, d_x.data_ptr(), d_y.data_ptr(), M,
                               1 if zp_int else 0, d_ws.data_ptr() if wsb else None, stream(torch)))
        torch.cuda.synchronize()
        got = d_y.double().cpu().numpy()
        assert np.all(np.isfinite(got))
        assert np.all(np.abs(got - want) <= 1e-2 * denom)
        assert np.percentile(np.abs(got - want) / denom, 99) <= 2.0 ** -9
        if wsb:
            assert int(d_ws[:4096].to(torch.int32).sum().item()) == 0


def test_gemm_one_hot_and_token_independence(awq, lib, torch_gpu):
    torch = torch_gpu
    m, k, M = 256, 512, 20
    scale = np.ones(m // 128, dtype=np.float16)
    zp = np.zeros(m // 128, dtype=np.float16)
    x = ((np.arange(M * k).reshape(M, k) % 13) + 1).astype(np.float16)
    for p, q in [(0, 5), (m + 1, 9), (3 * m + 17, 15), (k * m - 1, 1)]:
        packed = np.zeros(m * k // 2, dtype=np.uint8)
        packed[p >> 1] = q << (4 * (p & 1))
        d_in = dev(torch, packed)
        d_w = torch.zeros(m * k // 2, dtype=torch.uint8, device="cuda")
        awq.check(lib.awq_linear_repack(d_in.data_ptr(), d_w.data_ptr(), m, k, stream(torch)))
        d_s, d_z, d_x = dev(torch, scale), dev(torch, zp), dev(torch, x)
        d_y = torch.zeros((M, m), dtype=torch.float16, device="cuda")
        awq.check(lib.awq_gemm(d_w.data_ptr(), d_s.data_ptr(), d_z.data_ptr(), m, k, d_x.data_ptr(), d_y.data_ptr(), M,
                               1, None, stream(torch)))
        torch.cuda.synchronize()
        y = d_y.cpu().numpy().astype(np.float64)
        expect = np.zeros((M, m))
        expect[:, p % m] = q * x[:, p // m].astype(np.float64)
        assert np.array_equal(y, expect), p
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    b = buf.data_ptr()
    assert lib.awq_gemm(b, b, b, 128 * 37, 512, b, b, 4, 1, None, None) != 0   # input-dependent scale groups: refused
