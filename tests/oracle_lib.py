"""ctypes view of oracle/libawq_oracle.so (the CPU checker; test infrastructure)."""
import ctypes
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PATH = os.path.join(ROOT, "oracle", "libawq_oracle.so")

vp, i32, i64, u16, f32, f64 = (ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_uint16, ctypes.c_float,
                               ctypes.c_double)


class OracleConfig(ctypes.Structure):
    _fields_ = [("n_layers", ctypes.c_int), ("hidden", ctypes.c_int), ("inter", ctypes.c_int),
                ("vocab", ctypes.c_int), ("max_pos", ctypes.c_int), ("split_idx", ctypes.c_int),
                ("eps", ctypes.c_float)]


SIG = {
    "awqo_soft_h2f": (f32, [u16]),
    "awqo_soft_f2h": (u16, [f32]),
    "awqo_h2f": (f32, [u16]),
    "awqo_f2h": (u16, [f32]),
    "awqo_expf": (f32, [f32]),
    "awqo_erff": (f32, [f32]),
    "awqo_group_index": (ctypes.c_int, [i64, i64, i64, i64]),
    "awqo_group_period": (ctypes.c_int, [i64, i64]),
    "awqo_num_threads": (ctypes.c_int, []),
    "awqo_dequant": (None, [vp, vp, vp, vp, i64, i64, i64]),
    "awqo_linear_f64": (None, [vp, vp, vp, i64, i64, vp, vp, i64]),
    "awqo_linear_seq": (None, [vp, vp, vp, i64, i64, vp, vp, i64]),
    "awqo_linear_scalar": (None, [vp, vp, vp, i64, i64, vp, vp, i64]),
    "awqo_linear": (None, [vp, vp, vp, i64, i64, vp, vp, i64]),
    "awqo_rmsnorm": (None, [vp, vp, vp, i64, f32]),
    "awqo_rope_tables": (None, [vp, vp, i64]),
    "awqo_rotary": (None, [vp, vp, vp, ctypes.c_int, i64]),
    "awqo_kv_append": (None, [vp, vp, ctypes.c_int, i64, i64]),
    "awqo_attention": (None, [vp, vp, vp, vp, ctypes.c_int, i64, i64, vp]),
    "awqo_residual": (None, [vp, vp, vp, i64]),
    "awqo_gelu": (None, [vp, i64]),
    "awqo_argmax": (ctypes.c_int, [vp, i64]),
    "awqo_embed": (None, [vp, vp, vp, i64, i64, i64, vp]),
    "awqo_model_create": (vp, [ctypes.POINTER(OracleConfig)]),
    "awqo_model_destroy": (None, [vp]),
    "awqo_model_tensor": (vp, [vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(i64)]),
    "awqo_model_load_dir": (ctypes.c_int, [vp, ctypes.c_char_p]),
    "awqo_model_layer": (None, [vp, ctypes.c_int, i64, i64]),
    "awqo_model_sample": (ctypes.c_int, [vp]),
    "awqo_model_reset": (None, [vp]),
    "awqo_model_generate": (ctypes.c_int, [vp, vp, ctypes.c_int, ctypes.c_int, vp]),
    "awqo_model_hidden": (vp, [vp]),
    "awqo_model_logits": (vp, [vp]),
    "awqo_model_last_layer_out": (vp, [vp]),
    "awqo_model_hidden_mut": (vp, [vp]),
    "awqo_model_kcache": (vp, [vp, ctypes.c_int]),
    "awqo_model_vcache": (vp, [vp, ctypes.c_int]),
    "awqo_model_margins": (ctypes.c_int, [vp, vp, ctypes.c_int]),
    "awqo_model_seconds_linear": (f64, [vp]),
    "awqo_model_set_linear_mode": (None, [vp, ctypes.c_int]),
}

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(PATH):
            raise RuntimeError("oracle/libawq_oracle.so is not built: run `make -C oracle`")
        lib = ctypes.CDLL(PATH)
        for name, (res, args) in SIG.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib
