"""ctypes binding of libpkh3attn.so (declared in include/pkh3_attn.h).

The library is the only compute path: if it is missing, loading raises -- there is no fallback.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# PKH3_LIB_PATH selects another build of the same library (e.g. an experimental one); default: next to this file
LIB_PATH = os.environ.get("PKH3_LIB_PATH") or os.path.join(_HERE, "libpkh3attn.so")

PKH3_OK = 0
PKH3_ENULL = -1
PKH3_ESHAPE = -2
PKH3_EHEADDIM = -3
PKH3_ESTRIDE = -4
PKH3_EALIGN = -5
PKH3_EWORKSPACE = -6
PKH3_EUNSUPPORTED = -7
PKH3_EHIP = -8
PKH3_EARG = -9

ROPE_NONE, ROPE_INTERLEAVED, ROPE_HALF = 0, 1, 2
FLAG_FP8_QK = 1
FLAG_LONG_KEY_KERNEL = 2
FLAG_KV_PREPARED = 4
FLAG_O_IMAGES = 8
FLAG_FP8_POW2_SCALES = 16
NORM_NONE, NORM_LAYER, NORM_RMS = 0, 1, 2
LORA_RANK = 128  # PKH3_LORA_RANK
NOALLOC_SCRATCH_BYTES = 64 << 20  # PKH3_NOALLOC_SCRATCH_BYTES

EXPORTS = (
    "pkh3_workspace_bytes",
    "pkh3_attn_fwd",
    "pkh3_kv_prepare",
    "pkh3_attn_fwd_noalloc",
    "pkh3_noalloc_init",
    "pkh3_rope_tables",
    "pkh3_version",
    "pkh3_strerror",
    "pkh3_last_error",
    "pkh3_packed_bytes",
    "pkh3_pack_weight",
    "pkh3_pack_rows",
    "pkh3_adaln_modulate",
    "pkh3_qkv_proj",
    "pkh3_out_proj",
)


class AttnArgs(C.Structure):
    """Mirror of ``struct pkh3_attn_args``."""

    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
        ("q_sb", C.c_int64), ("q_ss", C.c_int64), ("q_sh", C.c_int64),
        ("k_sb", C.c_int64), ("k_ss", C.c_int64), ("k_sh", C.c_int64),
        ("v_sb", C.c_int64), ("v_ss", C.c_int64), ("v_sh", C.c_int64),
        ("o_sb", C.c_int64), ("o_ss", C.c_int64), ("o_sh", C.c_int64),
        ("B", C.c_int32), ("H", C.c_int32), ("Sq", C.c_int32), ("Sk", C.c_int32), ("D", C.c_int32),
        ("softmax_scale", C.c_float),
        ("q_norm_w", C.c_void_p), ("k_norm_w", C.c_void_p),
        ("norm_eps", C.c_float),
        ("rope_mode", C.c_int32),
        ("q_rope_cos", C.c_void_p), ("q_rope_sin", C.c_void_p),
        ("k_rope_cos", C.c_void_p), ("k_rope_sin", C.c_void_p),
        ("key_mask", C.c_void_p),
        ("blk_row_ptr", C.c_void_p), ("blk_col_idx", C.c_void_p),
        ("flags", C.c_uint32),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
    ]


class Linear(C.Structure):
    """Mirror of ``struct pkh3_linear``."""

    _fields_ = [
        ("w_img", C.c_void_p), ("bias", C.c_void_p),
        ("lora_a_img", C.c_void_p), ("lora_b_img", C.c_void_p),
        ("lora_scale", C.c_float),
    ]


class QkvArgs(C.Structure):
    """Mirror of ``struct pkh3_qkv_args``."""

    _fields_ = [
        ("x_img", C.c_void_p), ("S", C.c_int32), ("K", C.c_int32),
        ("q", Linear), ("k", Linear), ("v", Linear),
        ("lora_workspace", C.c_void_p), ("lora_workspace_bytes", C.c_size_t),
    ]


class OutArgs(C.Structure):
    """Mirror of ``struct pkh3_out_args``."""

    _fields_ = [
        ("o_img", C.c_void_p), ("S", C.c_int32), ("K", C.c_int32), ("N", C.c_int32),
        ("proj", Linear),
        ("gate", C.c_void_p), ("gate_stride", C.c_int64), ("row_index", C.c_void_p),
        ("residual", C.c_void_p), ("residual_stride", C.c_int64),
        ("y", C.c_void_p), ("y_stride", C.c_int64),
        ("lora_workspace", C.c_void_p), ("lora_workspace_bytes", C.c_size_t),
    ]


class Pkh3Error(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"libpkh3attn error {code}: {message}")
        self.code = code
        self.message = message


_lib = None


def load() -> C.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`); there is no fallback path"
        )
    lib = C.CDLL(LIB_PATH)
    lib.pkh3_workspace_bytes.argtypes = [C.POINTER(AttnArgs)]
    lib.pkh3_workspace_bytes.restype = C.c_size_t
    lib.pkh3_attn_fwd.argtypes = [C.POINTER(AttnArgs), C.c_void_p]
    lib.pkh3_attn_fwd.restype = C.c_int
    lib.pkh3_kv_prepare.argtypes = [C.POINTER(AttnArgs), C.c_void_p]
    lib.pkh3_kv_prepare.restype = C.c_int
    lib.pkh3_attn_fwd_noalloc.argtypes = [C.POINTER(AttnArgs), C.c_void_p]
    lib.pkh3_attn_fwd_noalloc.restype = C.c_int
    lib.pkh3_noalloc_init.argtypes = []
    lib.pkh3_noalloc_init.restype = C.c_int
    lib.pkh3_rope_tables.argtypes = [C.c_void_p, C.c_int32, C.POINTER(C.c_int32), C.c_double, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.pkh3_rope_tables.restype = C.c_int
    lib.pkh3_packed_bytes.argtypes = [C.c_int32, C.c_int32]
    lib.pkh3_packed_bytes.restype = C.c_size_t
    lib.pkh3_pack_weight.argtypes = [C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    lib.pkh3_pack_weight.restype = C.c_int
    lib.pkh3_pack_rows.argtypes = [C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    lib.pkh3_pack_rows.restype = C.c_int
    lib.pkh3_adaln_modulate.argtypes = [C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_float, C.c_void_p,
                                        C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.pkh3_adaln_modulate.restype = C.c_int
    lib.pkh3_qkv_proj.argtypes = [C.POINTER(QkvArgs), C.POINTER(AttnArgs), C.c_void_p]
    lib.pkh3_qkv_proj.restype = C.c_int
    lib.pkh3_out_proj.argtypes = [C.POINTER(OutArgs), C.c_void_p]
    lib.pkh3_out_proj.restype = C.c_int
    lib.pkh3_version.argtypes = []
    lib.pkh3_version.restype = C.c_int
    lib.pkh3_strerror.argtypes = [C.c_int]
    lib.pkh3_strerror.restype = C.c_char_p
    lib.pkh3_last_error.argtypes = []
    lib.pkh3_last_error.restype = C.c_char_p
    _lib = lib
    return lib


BENCH_LIB_PATH = os.path.join(os.path.dirname(LIB_PATH), "libpkh3attn_bench.so")
BENCH_EXPORTS = ("pkh3_attn_time_kernel",)   # include/pkh3_attn_bench.h
_bench = None


def load_bench() -> C.CDLL:
    """The measurement library (``libpkh3attn_bench.so``, the one call that synchronises with the device): for
    benchmark harnesses only, never loaded by the product path.  It links against the product library, which is
    loaded first so that both share one copy of it."""
    global _bench
    if _bench is not None:
        return _bench
    load()
    if not os.path.exists(BENCH_LIB_PATH):
        raise ImportError(f"{BENCH_LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}`")
    lib = C.CDLL(BENCH_LIB_PATH)
    lib.pkh3_attn_time_kernel.argtypes = [C.POINTER(AttnArgs), C.c_void_p, C.c_int, C.POINTER(C.c_float)]
    lib.pkh3_attn_time_kernel.restype = C.c_int
    _bench = lib
    return lib


def check(rc: int) -> None:
    if rc != PKH3_OK:
        lib = load()
        msg = lib.pkh3_last_error().decode() or lib.pkh3_strerror(rc).decode()
        raise Pkh3Error(rc, msg)
