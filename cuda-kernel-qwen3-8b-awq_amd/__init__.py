"""MI355X-native AWQ int4 decode engine: Python binding of the C ABI.

The package directory name contains hyphens; import it with
``importlib.import_module("cuda-kernel-qwen3-8b-awq_amd")``.

Everything here calls ``libawq_infer.so`` (HIP, gfx950).  There is no CPU
fallback: if the library is missing, loading fails and says how to build it.

``QWen3AWQInfer`` mirrors the reference class of the same name
(Inference.cu:356-366): ``QWen3AWQInfer(weight_dir)`` and
``generateResponse(prompt_ids, max_new_tokens)``.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libawq_infer.so")
INCLUDE_DIR = os.path.join(os.path.dirname(_HERE), "include")

# enum awq_tensor_kind / awq_tensor_part (include/awq_synth.h)
T_WQKV, T_WO, T_W1, T_W2, T_GAMMA, T_EMBED, T_UNEMBED = range(7)
P_PACKED, P_SCALE, P_ZP = range(3)
SYNTH_STREAM_INPUT = 0x100000
SYNTH_SPEC, SYNTH_BALANCED = 0, 1


class AwqConfig(ctypes.Structure):
    """struct awq_config; defaults are the constants of Inference.cu:33-47."""
    _fields_ = [
        ("n_layers", ctypes.c_int32),
        ("hidden", ctypes.c_int32),
        ("inter", ctypes.c_int32),
        ("vocab", ctypes.c_int32),
        ("max_pos", ctypes.c_int32),
        ("split_idx", ctypes.c_int32),
        ("eps", ctypes.c_float),
    ]

    def tensor_dims(self, kind):
        H, I, V = self.hidden, self.inter, self.vocab
        return {T_WQKV: (3 * H, H), T_WO: (H, H), T_W1: (I, H), T_W2: (H, I), T_EMBED: (H, V), T_UNEMBED: (V, H)}[kind]

    def part_count(self, kind, part):
        """number of elements (bytes for packed, halves otherwise) of one stored array"""
        if kind == T_GAMMA:
            return self.hidden
        o, i = self.tensor_dims(kind)
        return o * (i // 2) if part == P_PACKED else o // 128


_vp, _i32, _i64, _u64, _f32 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_uint64, ctypes.c_float
_cfgp = ctypes.POINTER(AwqConfig)

# name -> (restype, argtypes); every symbol declared in include/awq_infer.h
SIGNATURES = {
    "awq_last_error": (ctypes.c_char_p, []),
    "awq_default_config": (None, [_cfgp]),
    "awq_validate_weight_dir": (ctypes.c_int, [ctypes.c_char_p, _cfgp]),
    "awq_create": (ctypes.c_int, [ctypes.c_char_p, _cfgp, ctypes.POINTER(_vp)]),
    "awq_create_empty": (ctypes.c_int, [_cfgp, ctypes.POINTER(_vp)]),
    "awq_upload": (ctypes.c_int, [_vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, _i64]),
    "awq_finalize": (ctypes.c_int, [_vp]),
    "awq_generate": (ctypes.c_int, [_vp, _vp, _i32, _i32, _vp]),
    "awq_reset": (ctypes.c_int, [_vp]),
    "awq_prefill": (ctypes.c_int, [_vp, _vp, _i32]),
    "awq_decode": (ctypes.c_int, [_vp, _i32, _vp]),
    "awq_prefill_batched": (ctypes.c_int, [_vp, _vp, _i32]),
    "awq_set_prefill_mode": (ctypes.c_int, [_vp, ctypes.c_int]),
    "awq_debug_force_handover_giveup": (ctypes.c_int, [_vp, ctypes.c_int]),
    "awq_qkv_attention_workspace_bytes": (_i64, [ctypes.c_int32]),
    "awq_qkv_attention_supported": (ctypes.c_int, [_i64, ctypes.c_int32, _vp]),
    "awq_kv_parts_bytes": (_i64, [ctypes.c_int32, _i64]),
    "awq_kv_cache_to_parts": (ctypes.c_int, [_vp, _vp, _i64, ctypes.c_int32, _vp, _vp, _i64, _i64, _i64, _vp]),
    "awq_qkv_attention": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _i64,
                                         ctypes.c_int32, _i64, _i64, _vp, _vp, _vp, ctypes.c_int32, _vp]),
    "awq_qkv_attention_status": (ctypes.c_int, [_vp, _vp]),
    "awq_set_fused_mode": (ctypes.c_int, [_vp, ctypes.c_int]),
    "awq_fused_mode": (ctypes.c_int, [_vp]),
    "awq_debug_fused_timeline": (ctypes.c_int, [_vp, ctypes.c_int32, _vp, _vp, _vp]),
    "awq_debug_qkv_attention_timeline": (ctypes.c_int, [_vp, ctypes.c_int32, ctypes.c_int32, _vp, _vp, _vp]),
    "awq_read_hidden": (ctypes.c_int, [_vp, _vp]),
    "awq_read_logits": (ctypes.c_int, [_vp, _vp]),
    "awq_set_graph_mode": (ctypes.c_int, [_vp, ctypes.c_int]),
    "awq_time_linear": (ctypes.c_int, [_vp, ctypes.c_int, _i32, ctypes.POINTER(_f32), ctypes.POINTER(_i64)]),
    "awq_destroy": (None, [_vp]),
    "awq_write_weight_dir": (ctypes.c_int, [ctypes.c_char_p, _cfgp, _u64]),
    "awq_write_weight_dir_profile": (ctypes.c_int, [ctypes.c_char_p, _cfgp, _u64, ctypes.c_int]),
    "awq_last_load_seconds": (ctypes.c_double, []),
    "awq_synth_fill": (ctypes.c_int, [_u64, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, _i64]),
    "awq_synth_fill_profile": (ctypes.c_int, [ctypes.c_int, _u64, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, _i64]),
    "awq_synth_normal_f16": (ctypes.c_int, [_u64, _u64, _vp, _i64, _f32, _f32]),
    "awq_synth_tokens": (ctypes.c_int, [_u64, _u64, _vp, _i64, _i32]),
    "awq_rope_tables_host": (ctypes.c_int, [_vp, _vp, _i64]),
    "awq_dequant": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "awq_linear_repack": (ctypes.c_int, [_vp, _vp, _i64, _i64, _vp]),
    "awq_gemv_workspace_bytes": (_i64, [_i64, _i64]),
    "awq_gemv": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp]),
    "awq_gemm_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "awq_gemm_plan": (_i32, [_i64, _i64, _i64, _i32]),
    "awq_gemm": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i64, _vp, _vp, _i64, _i32, _vp, _vp]),
    "awq_rmsnorm": (ctypes.c_int, [_vp, _vp, _vp, _i64, _f32, _vp]),
    "awq_rope_kv_append": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp]),
    "awq_attention_workspace_bytes": (_i64, [_i32, _i64]),
    "awq_decode_attention": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp, _vp]),
    "awq_decode_attention_static": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp]),
    "awq_prefill_attention": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32, _i64, _i64, _i64, _i32, _vp]),
    "awq_residual_add": (ctypes.c_int, [_vp, _vp, _vp, _i64, _vp]),
    "awq_gelu": (ctypes.c_int, [_vp, _i64, _vp]),
    "awq_argmax_workspace_bytes": (_i64, [_i64]),
    "awq_logits_argmax": (ctypes.c_int, [_vp, _i64, _vp, _vp, _vp]),
    "awq_embed_gather": (ctypes.c_int, [_vp, _vp, _vp, _i64, _i64, _i32, _vp, _vp]),
}



class AwqLinearArgs(ctypes.Structure):
    """struct awq_linear_args"""
    _fields_ = [
        ("repacked", _vp), ("scale", _vp), ("zp", _vp), ("m", _i64), ("k", _i64), ("x", _vp), ("y", _vp),
        ("reserved0", _i32), ("prologue", _i32), ("epilogue", _i32), ("eps", _f32), ("gamma", _vp),
        ("residual", _vp), ("cos_t", _vp), ("sin_t", _vp), ("k_cache", _vp), ("v_cache", _vp), ("hidden", _i32),
        ("reserved", _i32), ("max_pos", _i64), ("pos", _i64), ("out_token", _vp), ("workspace", _vp),
    ]


PRO_NONE, PRO_RMSNORM = 0, 1
EPI_STORE, EPI_RESIDUAL, EPI_GELU, EPI_QKV_ROPE, EPI_ARGMAX = range(5)
SIGNATURES["awq_gemv_fused"] = (ctypes.c_int, [ctypes.POINTER(AwqLinearArgs), _vp])

_lib = None


def load_library():
    """Load libawq_infer.so and attach the signatures.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libawq_infer.so is not built: run `python %s` (needs hipcc); there is no CPU fallback"
            % os.path.join(_HERE, "build.py"))
    # PyTorch (used by callers for device memory and streams) bundles its own HIP runtime.  Two
    # HIP runtimes in one process cannot both own the GPU, so torch is imported first: the loader
    # then resolves this library's libamdhip64.so.7 to the copy that is already mapped.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class AwqError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("awq error %d: %s" % (code, message))
        self.code = code


def check(rc):
    if rc != 0:
        raise AwqError(rc, load_library().awq_last_error().decode("utf-8", "replace"))


def default_config():
    cfg = AwqConfig()
    load_library().awq_default_config(ctypes.byref(cfg))
    return cfg


def make_config(n_layers=36, hidden=4096, inter=12288, vocab=151936, max_pos=40960, split_idx=None, eps=1e-6):
    if split_idx is None:
        split_idx = n_layers // 2  # Inference.cu:47
    return AwqConfig(n_layers, hidden, inter, vocab, max_pos, split_idx, eps)


def _int32_array(values):
    arr = (ctypes.c_int32 * max(1, len(values)))()
    for i, v in enumerate(values):
        arr[i] = int(v)
    return arr


class QWen3AWQInfer:
    """The reference's engine class (Inference.cu:356-366) on one MI355X.

    ``QWen3AWQInfer(weight_dir)`` loads the reference's .bin directory
    (Inference.cu:780-899); ``config`` overrides the model constants (tests).
    Errors raise ``AwqError`` (the C++ class of the same name keeps the
    reference's print-and-exit(1)).
    """

    def __init__(self, weight_dir=None, config=None, _handle=None):
        self._lib = load_library()
        self._h = _vp()
        self.config = config if config is not None else default_config()
        if _handle is not None:
            self._h = _handle
            return
        if weight_dir is None:
            raise ValueError("weight_dir is required (or use QWen3AWQInfer.empty / from_synthetic)")
        check(self._lib.awq_create(os.fsencode(weight_dir), ctypes.byref(self.config), ctypes.byref(self._h)))

    @classmethod
    def empty(cls, config):
        """An engine that waits for upload() of every array and then finalize()."""
        lib = load_library()
        h = _vp()
        check(lib.awq_create_empty(ctypes.byref(config), ctypes.byref(h)))
        return cls(config=config, _handle=h)

    @classmethod
    def from_synthetic(cls, config, seed, keep_host=None):
        """Fill every tensor from the seeded generator (include/awq_synth.h).

        keep_host: optional callable (layer, kind, part, ctypes_buffer) that sees
        each host array before it is dropped (tests hand them to the checker).
        """
        eng = cls.empty(config)
        lib = eng._lib
        for layer, kind, part in tensor_list(config):
            count = config.part_count(kind, part)
            nbytes = count if (part == P_PACKED and kind != T_GAMMA) else 2 * count
            buf = (ctypes.c_uint8 * nbytes)()
            check(lib.awq_synth_fill(seed, layer, kind, part, buf, count))
            if keep_host is not None:
                keep_host(layer, kind, part, buf)
            check(lib.awq_upload(eng._h, layer, kind, part, buf, nbytes))
        eng.finalize()
        return eng

    def upload(self, layer, kind, part, host_ptr, nbytes):
        check(self._lib.awq_upload(self._h, layer, kind, part, host_ptr, nbytes))

    def finalize(self):
        check(self._lib.awq_finalize(self._h))

    def generateResponse(self, prompt_ids, max_new_tokens):
        """Returns only the newly generated token ids (Inference.cu:361-366)."""
        prompt = _int32_array(prompt_ids)
        out = (ctypes.c_int32 * max(1, max_new_tokens))()
        check(self._lib.awq_generate(self._h, prompt, len(prompt_ids), max_new_tokens, out))
        return [int(out[i]) for i in range(max_new_tokens)]

    # the same loop in pieces (timing)
    def reset(self):
        check(self._lib.awq_reset(self._h))

    def prefill(self, prompt_ids, batched=False):
        """The prompt loop; batched=True sends all positions through each layer together."""
        fn = self._lib.awq_prefill_batched if batched else self._lib.awq_prefill
        check(fn(self._h, _int32_array(prompt_ids), len(prompt_ids)))

    def set_prefill_mode(self, batched):
        """Which prompt loop generateResponse uses (default: token by token)."""
        check(self._lib.awq_set_prefill_mode(self._h, 1 if batched else 0))

    def decode(self, n_steps):
        out = (ctypes.c_int32 * max(1, n_steps))()
        check(self._lib.awq_decode(self._h, n_steps, out))
        return [int(out[i]) for i in range(n_steps)]

    FUSED_WO_W1 = 1      # Wo + residual and RMSNorm + W1 + GeLU of a layer as one launch
    FUSED_QKV_ATTN = 2   # RMSNorm + Wqkv + rotary + KV append and the attention of a layer as one launch

    def set_fused_mode(self, mode):
        """Which pairs of a layer's launches run as one (a sum of FUSED_*; True means FUSED_WO_W1, False or 0
        none).  A pair the device cannot run fused stays two launches: fused_mode() tells what is on."""
        check(self._lib.awq_set_fused_mode(self._h, int(mode)))

    def fused_mode(self):
        return int(self._lib.awq_fused_mode(self._h))

    def set_graph_mode(self, enabled):
        check(self._lib.awq_set_graph_mode(self._h, 1 if enabled else 0))

    def read_hidden(self):
        buf = (ctypes.c_uint16 * self.config.hidden)()
        check(self._lib.awq_read_hidden(self._h, buf))
        return buf

    def read_logits(self):
        buf = (ctypes.c_uint16 * self.config.vocab)()
        check(self._lib.awq_read_logits(self._h, buf))
        return buf

    def time_linear(self, kind, n_rounds=20):
        """(mean microseconds per launch, algorithmic bytes per launch) of the fused linear kernel"""
        us, nbytes = _f32(0), _i64(0)
        check(self._lib.awq_time_linear(self._h, kind, n_rounds, ctypes.byref(us), ctypes.byref(nbytes)))
        return us.value, nbytes.value

    def close(self):
        if self._h:
            self._lib.awq_destroy(self._h)
            self._h = _vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def tensor_list(config):
    """(layer, kind, part) of every stored array, in the loader's order (Inference.cu:766-903)."""
    out = []
    for l in range(config.n_layers):
        for kind in (T_WQKV, T_WO, T_W1, T_W2):
            for part in (P_PACKED, P_SCALE, P_ZP):
                out.append((l, kind, part))
        out.append((l, T_GAMMA, 0))
    for kind in (T_EMBED, T_UNEMBED):
        for part in (P_PACKED, P_SCALE, P_ZP):
            out.append((0, kind, part))
    return out
