"""C-ABI checks that need no GPU: the library loads, exports every symbol include/pkh3_attn.h
declares, and rejects bad arguments on the host before any HIP call."""
import ctypes as C
import os
import re

import pytest

import pika_h3_flex_amd as pk
from pika_h3_flex_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_are_exported(lib):
    inc = os.path.join(ROOT, "include")
    header = "".join(open(os.path.join(inc, f)).read() for f in sorted(os.listdir(inc)) if f.endswith(".h"))
    declared = set(re.findall(r"\b(pkh3_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    for name in declared:
        assert getattr(lib, name) is not None


def test_version_and_strerror(lib):
    assert lib.pkh3_version() == 102
    assert lib.pkh3_strerror(0) == b"ok"
    assert b"128" in lib.pkh3_strerror(_lib.PKH3_EHEADDIM)


def test_struct_layout_matches_header():
    """Field order and count of the ctypes mirror follow struct pkh3_attn_args in the header."""
    header = open(os.path.join(ROOT, "include", "pkh3_attn.h")).read()
    body = header[header.index("typedef struct pkh3_attn_args {"): header.index("} pkh3_attn_args;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split("{", 1)[1].split(";"):
        decl = decl.strip()
        if not decl:
            continue
        for part in decl.split(","):
            names.append(re.findall(r"[A-Za-z_][A-Za-z_0-9]*", part)[-1])
    assert names == [f[0] for f in _lib.AttnArgs._fields_]


def _valid_args():
    a = _lib.AttnArgs()
    buf = 0x10000  # fake, aligned device addresses: validation never dereferences them
    a.q = a.k = a.v = a.o = buf
    for n in ("q", "k", "v", "o"):
        setattr(a, n + "_sb", 64 * 2 * 128)
        setattr(a, n + "_ss", 2 * 128)
        setattr(a, n + "_sh", 128)
    a.B, a.H, a.Sq, a.Sk, a.D = 1, 2, 64, 64, 128
    a.norm_eps = 1e-6
    a.workspace = 0x100000
    a.workspace_bytes = 1 << 30
    return a


def test_workspace_bytes_host_only(lib):
    a = _valid_args()
    n = lib.pkh3_workspace_bytes(C.byref(a))
    # one [K|V] tile record per head (Q is consumed in place)
    assert 2 * 32768 <= n < 2 * 32768 + 4096 and n % 256 == 0
    a.flags = _lib.FLAG_FP8_QK
    n8 = lib.pkh3_workspace_bytes(C.byref(a))
    assert 0 < n8 < n
    a.D = 64
    assert lib.pkh3_workspace_bytes(C.byref(a)) == 0


@pytest.mark.parametrize("mutate,code", [
    (lambda a: setattr(a, "D", 64), _lib.PKH3_EHEADDIM),
    (lambda a: setattr(a, "q", 0), _lib.PKH3_ENULL),
    (lambda a: setattr(a, "Sq", 0), _lib.PKH3_ESHAPE),
    (lambda a: setattr(a, "H", 70000), _lib.PKH3_ESHAPE),
    (lambda a: setattr(a, "k", 0x10008), _lib.PKH3_EALIGN),
    (lambda a: setattr(a, "v_ss", 132), _lib.PKH3_ESTRIDE),
    (lambda a: setattr(a, "o_sh", -128), _lib.PKH3_ESTRIDE),
    (lambda a: setattr(a, "workspace", 0), _lib.PKH3_EWORKSPACE),
    (lambda a: setattr(a, "workspace", 0x100010), _lib.PKH3_EWORKSPACE),
    (lambda a: setattr(a, "workspace_bytes", 1024), _lib.PKH3_EWORKSPACE),
    (lambda a: setattr(a, "flags", 0x80), _lib.PKH3_EARG),
    (lambda a: setattr(a, "rope_mode", 7), _lib.PKH3_EARG),
    (lambda a: setattr(a, "rope_mode", 1), _lib.PKH3_ENULL),          # tables missing
    (lambda a: setattr(a, "blk_row_ptr", 0x20000), _lib.PKH3_ENULL),  # col_idx missing
    (lambda a: (setattr(a, "blk_row_ptr", 0x20000), setattr(a, "blk_col_idx", 0x30000), setattr(a, "key_mask", 0x40000)),
     _lib.PKH3_EUNSUPPORTED),
    (lambda a: (setattr(a, "flags", 1), setattr(a, "key_mask", 0x40000)), _lib.PKH3_EUNSUPPORTED),
    (lambda a: setattr(a, "softmax_scale", float("nan")), _lib.PKH3_EARG),
])
def test_argument_errors_are_reported_before_any_launch(lib, mutate, code):
    a = _valid_args()
    mutate(a)
    rc = lib.pkh3_attn_fwd(C.byref(a), None)
    assert rc == code
    assert lib.pkh3_last_error() != b""
    with pytest.raises(_lib.Pkh3Error) as ei:
        _lib.check(rc)
    assert ei.value.code == code


def test_null_args_pointer(lib):
    assert lib.pkh3_attn_fwd(None, None) == _lib.PKH3_ENULL
    assert lib.pkh3_workspace_bytes(None) == 0


def test_rope_tables_argument_errors(lib):
    dims = (C.c_int32 * 3)(32, 48, 48)
    assert lib.pkh3_rope_tables(None, 4, dims, 1e4, 0x1000, 0x2000, None) == _lib.PKH3_ENULL
    assert lib.pkh3_rope_tables(0x1000, 0, dims, 1e4, 0x1000, 0x2000, None) == _lib.PKH3_ESHAPE
    bad = (C.c_int32 * 3)(32, 48, 40)
    assert lib.pkh3_rope_tables(0x1000, 4, bad, 1e4, 0x1000, 0x2000, None) == _lib.PKH3_EARG
    odd = (C.c_int32 * 3)(31, 49, 48)
    assert lib.pkh3_rope_tables(0x1000, 4, odd, 1e4, 0x1000, 0x2000, None) == _lib.PKH3_EARG


def test_time_kernel_argument_errors(lib):
    a = _valid_args()
    assert lib.pkh3_attn_time_kernel(C.byref(a), None, 1, None) == _lib.PKH3_ENULL
    ms = C.c_float()
    assert lib.pkh3_attn_time_kernel(C.byref(a), None, 0, C.byref(ms)) == _lib.PKH3_EARG


def test_noalloc_entry_point_validates_on_the_host(lib):
    """pkh3_attn_fwd_noalloc ignores the caller's workspace fields, checks everything else like pkh3_attn_fwd,
    and rejects a call whose scratch would not fit its built-in buffer -- all before any HIP call."""
    a = _valid_args()
    a.q = 0
    assert lib.pkh3_attn_fwd_noalloc(C.byref(a), None) == _lib.PKH3_ENULL
    a = _valid_args()
    a.D = 64
    assert lib.pkh3_attn_fwd_noalloc(C.byref(a), None) == _lib.PKH3_EHEADDIM
    a = _valid_args()
    a.workspace, a.workspace_bytes = 0, 0       # not an error here
    a.H, a.Sk = 24, 8192                        # 24 x 128 tiles x 32 KiB = 96 MiB of K/V images
    for n in ("q", "k", "v", "o"):
        setattr(a, n + "_ss", 24 * 128)
    assert lib.pkh3_workspace_bytes(C.byref(a)) > _lib.NOALLOC_SCRATCH_BYTES
    assert lib.pkh3_attn_fwd_noalloc(C.byref(a), None) == _lib.PKH3_EWORKSPACE
    assert b"built-in" in lib.pkh3_last_error()
    header = open(os.path.join(ROOT, "include", "pkh3_attn.h")).read()
    assert re.search(r"#define\s+PKH3_NOALLOC_SCRATCH_BYTES\s+\(64u\s*<<\s*20\)", header)


def test_front_end_checks_every_pointer_for_its_device():
    """Tensors handed over by address (norm weights, rope tables, masks) must live where the kernels run."""
    import torch

    from pika_h3_flex_amd import ops

    host = torch.ones(128)
    with pytest.raises(ValueError, match="device memory"):
        ops._f32("q_norm_weight", host, (128,), torch.device("meta"))
    assert ops._f32("w", host, (128,), torch.device("cpu")) is host
    with pytest.raises(ValueError, match="contiguous float32"):
        ops._f32("w", host.double(), (128,), torch.device("cpu"))
    with pytest.raises(ValueError, match="device memory"):
        ops._on_device("key_mask", torch.zeros(4, dtype=torch.bool), torch.device("meta"))
    bm = ops.BlockMask.from_dense(torch.ones((2, 3), dtype=torch.bool), device="cpu")
    assert bm.n_cols == 3


def test_ops_refuse_host_tensors():
    """The product path never computes on the CPU: host tensors are an error, not a fallback."""
    import torch

    q = torch.zeros((1, 8, 2, 128), dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="device memory"):
        pk.attention(q, q, q)
    with pytest.raises(ValueError, match="device memory"):
        pk.rope_tables(torch.zeros((4, 3), dtype=torch.float64))


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libpkh3attn.so"))
    with pytest.raises(ImportError, match="no fallback"):
        _lib.load()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "pika-h3-flex_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"
