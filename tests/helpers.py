"""numpy utilities shared by the tests: pointer plumbing, an independent numpy
version of the seeded generator, reference packing helpers."""
import ctypes

import numpy as np

MASK64 = (1 << 64) - 1


def ptr(a):
    """void* of a contiguous numpy array"""
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


def f16(bits):
    return np.asarray(bits, dtype=np.uint16).view(np.float16)


def bits16(x):
    return np.asarray(x, dtype=np.float16).view(np.uint16)


# ---- independent numpy statement of include/awq_synth.h ----------------------
def synth_hash(seed, sid, idx):
    idx = np.asarray(idx, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = (np.uint64((seed * 0x9E3779B97F4A7C15) & MASK64) + np.uint64(((sid + 1) * 0xD1B54A32D192ED03) & MASK64)
             + idx * np.uint64(0xA0761D6478BD642F))
        z ^= z >> np.uint64(30)
        z *= np.uint64(0xBF58476D1CE4E5B9)
        z ^= z >> np.uint64(27)
        z *= np.uint64(0x94D049BB133111EB)
        z ^= z >> np.uint64(31)
    return z


def synth_stream(layer, kind, part):
    l = 0 if kind in (5, 6) else layer + 1
    return l * 64 + kind * 4 + part


def synth_packed(seed, layer, kind, nbytes):
    words = synth_hash(seed, synth_stream(layer, kind, 0), np.arange((nbytes + 7) // 8, dtype=np.uint64))
    return words.view(np.uint8)[:nbytes].copy()  # little endian host


def synth_scale(seed, layer, kind, n):
    h = synth_hash(seed, synth_stream(layer, kind, 1), np.arange(n, dtype=np.uint64))
    u = (h >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / 16777216.0)
    return (np.float32(0.002) + np.float32(0.018) * u).astype(np.float16)


def synth_zp(seed, layer, kind, n):
    h = synth_hash(seed, synth_stream(layer, kind, 2), np.arange(n, dtype=np.uint64))
    return (h & np.uint64(15)).astype(np.float32).astype(np.float16)


def synth_normal(seed, sid, n):
    idx = np.arange(n, dtype=np.uint64)
    a = synth_hash(seed, sid, idx * np.uint64(2))
    b = synth_hash(seed, sid, idx * np.uint64(2) + np.uint64(1))
    u1 = ((a >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
    u2 = (b >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(6.283185307179586 * u2)


# ---- AWQ helpers --------------------------------------------------------------
def nibbles_flat(packed):
    """flat nibble stream: low nibble first (Inference.cu:95-99)"""
    p = np.asarray(packed, dtype=np.uint8)
    out = np.empty(p.size * 2, dtype=np.uint8)
    out[0::2] = p & 15
    out[1::2] = p >> 4
    return out


def dequant_numpy(packed, scale, zp, rows, cols, n_groups):
    """(q - z) * s with binary16 rounding after each op, via numpy float16 arithmetic"""
    q = nibbles_flat(packed).reshape(rows, cols).astype(np.float16)
    g = (np.arange(cols) // 128) % n_groups
    sub = (q - zp[g][None, :]).astype(np.float16)
    return (sub * scale[g][None, :]).astype(np.float16)


def effective_weights_f64(packed, scale, zp, m, k):
    """W_eff[i, j] = dequantised flat element j*m + i (column-major read, Inference.cu:1059)"""
    flat = dequant_numpy(packed, scale, zp, m, k, m // 128).reshape(-1)
    return flat.astype(np.float64).reshape(k, m).T


def unrounded_weights_f64(packed, scale, zp, m, k):
    """W[i, j] = (q - z) * s in float64 for flat element j*m + i: the weights the blocked order of
    awq_canon_math.h multiplies (scale and zero-point applied to a block's sum, no binary16 rounding
    of each weight)"""
    q = nibbles_flat(packed).reshape(m, k).astype(np.float64)
    g = (np.arange(k) // 128) % (m // 128)
    flat = ((q - zp.astype(np.float64)[g][None, :]) * scale.astype(np.float64)[g][None, :]).reshape(-1)
    return flat.reshape(k, m).T


def block_elem(k, C, blk, t):
    U = k // (32 * C)
    c, u = divmod(blk, U)
    return c + C * (32 * u + t)


def repack_numpy(packed, m, k, C):
    """numpy statement of the streaming order of the GPU kernels (see csrc/gemv.hip):
    [row group of 16][block][row % 16][4 dwords]"""
    nib = nibbles_flat(packed).astype(np.uint32)
    nblk = k // 32
    out = np.zeros((m // 16, nblk, 16, 4), dtype=np.uint32)
    rows = np.arange(m).reshape(m // 16, 16)
    for blk in range(nblk):
        for t in range(32):
            j = block_elem(k, C, blk, t)
            q = nib[j * m + rows]
            tt = t & 7
            pos = (tt >> 1) * 4 + (tt & 1) * 16
            out[:, blk, :, t >> 3] |= q << np.uint32(pos)
    return out.reshape(-1)


# ---- engine / oracle pairs ----------------------------------------------------
def make_oracle_model(oracle, cfg):
    import oracle_lib
    ocfg = oracle_lib.OracleConfig(cfg.n_layers, cfg.hidden, cfg.inter, cfg.vocab, cfg.max_pos, cfg.split_idx, cfg.eps)
    return oracle.awqo_model_create(ctypes.byref(ocfg))


def fill_pair(awq, oracle, cfg, seed, engine=None, model=None, profile=0, mutate=None):
    """Fill the oracle model's host arrays from the seeded generator and upload the very same
    bytes to the engine.  mutate(layer, kind, part, address, count) may change a tensor in place
    before it is uploaded."""
    lib = awq.load_library()
    for layer, kind, part in awq.tensor_list(cfg):
        count = cfg.part_count(kind, part)
        nbytes = count if (part == awq.P_PACKED and kind != awq.T_GAMMA) else 2 * count
        got = ctypes.c_int64(0)
        p = oracle.awqo_model_tensor(model, layer, kind, part, ctypes.byref(got))
        assert got.value == nbytes, (layer, kind, part, got.value, nbytes)
        awq.check(lib.awq_synth_fill_profile(profile, seed, layer, kind, part, p, count))
        if mutate is not None:
            mutate(layer, kind, part, p, count)
        if engine is not None:
            engine.upload(layer, kind, part, p, nbytes)
    if engine is not None:
        engine.finalize()


# ---- activation shapes that stress the block fixed point of the linear layers ------------------
def heavy_tailed_inputs(rng, k):
    """name -> binary16 input vector of length k.  The linear layers round each input to 2^-16 of the largest
    magnitude in its block of 32, so what matters is how the magnitudes inside a block are spread."""
    out = {}
    x = rng.standard_normal(k)
    idx = 32 * np.arange(k // 32) + rng.integers(0, 32, size=k // 32)
    x[idx] = 1024.0 * np.where(rng.random(k // 32) < 0.5, -1.0, 1.0)
    out["one 2^10 outlier per block over N(0,1)"] = x.astype(np.float16)
    x = 1e-3 * rng.standard_normal(k)
    x[rng.choice(k, size=3, replace=False)] = np.array([3000.0, -2500.0, 1800.0])
    out["three massive channels over 1e-3 noise"] = x.astype(np.float16)
    out["Student-t, 2 degrees of freedom"] = np.clip(rng.standard_t(2, size=k), -60000, 60000).astype(np.float16)
    from math import erf
    g = rng.standard_normal(k)
    out["GeLU of N(0,1)"] = np.array([0.5 * v * (1.0 + erf(v * 0.70710678)) for v in g]).astype(np.float16)
    return out
