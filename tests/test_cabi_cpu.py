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
    assert declared == set(_lib.EXPORTS) | set(_lib.BENCH_EXPORTS), declared ^ (set(_lib.EXPORTS) | set(_lib.BENCH_EXPORTS))
    for name in _lib.EXPORTS:
        assert getattr(lib, name) is not None
    # the call that synchronises lives in the measurement library, not in the product library
    bench = _lib.load_bench()
    for name in _lib.BENCH_EXPORTS:
        assert getattr(bench, name) is not None
        assert not hasattr(lib, name)


def test_version_and_strerror(lib):
    assert lib.pkh3_version() == 107
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
    # 32-bit workgroup counts: B * H * ceil(Sq / 32) is bounded
    (lambda a: (setattr(a, "B", 60000), setattr(a, "H", 60000), setattr(a, "Sq", 1 << 20)), _lib.PKH3_ESHAPE),
    (lambda a: setattr(a, "k", 0x10008), _lib.PKH3_EALIGN),
    (lambda a: setattr(a, "v_ss", 132), _lib.PKH3_ESTRIDE),
    (lambda a: setattr(a, "o_sh", -128), _lib.PKH3_ESTRIDE),
    (lambda a: setattr(a, "workspace", 0), _lib.PKH3_EWORKSPACE),
    (lambda a: setattr(a, "workspace", 0x100010), _lib.PKH3_EWORKSPACE),
    (lambda a: setattr(a, "workspace_bytes", 1024), _lib.PKH3_EWORKSPACE),
    (lambda a: setattr(a, "flags", 0x80), _lib.PKH3_EARG),
    (lambda a: setattr(a, "flags", _lib.FLAG_FP8_POW2_SCALES), _lib.PKH3_EARG),   # an option of FLAG_FP8_QK only
    (lambda a: setattr(a, "rope_mode", 7), _lib.PKH3_EARG),
    (lambda a: setattr(a, "rope_mode", 1), _lib.PKH3_ENULL),          # tables missing
    (lambda a: setattr(a, "blk_row_ptr", 0x20000), _lib.PKH3_ENULL),  # col_idx missing
    (lambda a: (setattr(a, "blk_row_ptr", 0x20000), setattr(a, "blk_col_idx", 0x30000), setattr(a, "key_mask", 0x40000)),
     _lib.PKH3_EUNSUPPORTED),
    (lambda a: (setattr(a, "flags", 1), setattr(a, "key_mask", 0x40000)), _lib.PKH3_EUNSUPPORTED),
    (lambda a: setattr(a, "softmax_scale", float("nan")), _lib.PKH3_EARG),
    # output as operand images: one document only; the strides are not looked at, the pointer is
    (lambda a: (setattr(a, "flags", _lib.FLAG_O_IMAGES), setattr(a, "B", 2)), _lib.PKH3_EUNSUPPORTED),
    (lambda a: (setattr(a, "flags", _lib.FLAG_O_IMAGES), setattr(a, "o", 0)), _lib.PKH3_ENULL),
    (lambda a: (setattr(a, "flags", _lib.FLAG_O_IMAGES), setattr(a, "o", 0x10008)), _lib.PKH3_EALIGN),
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


def test_time_kernel_argument_errors():
    lib = _lib.load_bench()
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


# ---- projection entry points: host-side validation, no GPU ---------------------------------------------------
def test_packed_bytes_host_only(lib):
    assert lib.pkh3_packed_bytes(1, 32) == 256 * 32 * 2                  # rows padded to 256
    assert lib.pkh3_packed_bytes(48360, 3072) == 48384 * 3072 * 2
    assert lib.pkh3_packed_bytes(256, 4096) == 256 * 4096 * 2
    for rows, k in ((0, 64), (8, 0), (8, 48), (8, 4128), (-1, 64)):
        assert lib.pkh3_packed_bytes(rows, k) == 0


def test_pack_and_modulate_argument_errors(lib):
    x, out = 0x10000, 0x200000
    assert lib.pkh3_pack_rows(None, 64, 8, 64, out, None) == _lib.PKH3_ENULL
    assert lib.pkh3_pack_rows(x, 64, 8, 64, None, None) == _lib.PKH3_ENULL
    assert lib.pkh3_pack_rows(x + 2, 64, 8, 64, out, None) == _lib.PKH3_EALIGN
    assert lib.pkh3_pack_rows(x, 64, 8, 64, out + 16, None) == _lib.PKH3_EALIGN      # destination: 256-byte aligned
    assert lib.pkh3_pack_rows(x, 64, 0, 64, out, None) == _lib.PKH3_ESHAPE
    assert lib.pkh3_pack_rows(x, 64, 8, 48, out, None) == _lib.PKH3_ESHAPE           # K multiple of 32
    assert lib.pkh3_pack_rows(x, 8192, 8, 8192, out, None) == _lib.PKH3_ESHAPE       # K <= 4096
    assert lib.pkh3_pack_rows(x, 32, 8, 64, out, None) == _lib.PKH3_ESTRIDE          # stride < K
    assert lib.pkh3_pack_rows(x, 68, 8, 64, out, None) == _lib.PKH3_ESTRIDE          # stride not a multiple of 8
    assert lib.pkh3_pack_weight(x, 64, 100, 64, 1, out, None) == _lib.PKH3_ESHAPE    # whole 128-feature heads
    assert b"128" in lib.pkh3_last_error()
    mod = lib.pkh3_adaln_modulate
    assert mod(x, 64, 8, 64, 7, 1e-6, None, None, 0, None, out, None) == _lib.PKH3_EARG               # norm kind
    assert mod(x, 64, 8, 64, _lib.NORM_LAYER, float("nan"), None, None, 0, None, out, None) == _lib.PKH3_EARG
    assert mod(x, 64, 8, 64, _lib.NORM_NONE, 0.0, 0x30000, None, 64, None, out, None) == _lib.PKH3_EUNSUPPORTED
    assert mod(x, 64, 8, 64, _lib.NORM_LAYER, 1e-6, 0x30002, None, 64, None, out, None) == _lib.PKH3_EALIGN
    assert mod(x, 64, 8, 64, _lib.NORM_LAYER, 1e-6, 0x30000, None, 32, None, out, None) == _lib.PKH3_ESTRIDE


def _qkv_args():
    a = _valid_args()
    a.B, a.H, a.Sq, a.Sk = 1, 2, 64, 64
    p = _lib.QkvArgs()
    p.x_img, p.S, p.K = 0x400000, 64, 256
    for lin in (p.q, p.k, p.v):
        lin.w_img = 0x500000
    return p, a


def test_qkv_proj_argument_errors(lib):
    p, a = _qkv_args()
    assert lib.pkh3_qkv_proj(None, C.byref(a), None) == _lib.PKH3_ENULL
    assert lib.pkh3_qkv_proj(C.byref(p), None, None) == _lib.PKH3_ENULL
    p, a = _qkv_args(); a.k = a.v = 0                                    # K and V inputs are not needed
    a.B = 2
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_EUNSUPPORTED
    p, a = _qkv_args(); a.key_mask = 0x40000
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_EUNSUPPORTED
    p, a = _qkv_args(); a.Sk = 128
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_EUNSUPPORTED
    p, a = _qkv_args(); p.S = 65
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_ESHAPE
    p, a = _qkv_args(); p.K = 100
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_ESHAPE
    p, a = _qkv_args(); p.x_img = 0
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_ENULL
    p, a = _qkv_args(); p.k.w_img = 0
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_ENULL
    p, a = _qkv_args(); p.v.lora_a_img = 0x600000                        # A without B
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_ENULL
    p, a = _qkv_args(); p.v.lora_a_img = p.v.lora_b_img = 0x600000       # adapter without its scratch
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_EWORKSPACE
    p, a = _qkv_args(); a.workspace_bytes = 1024
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_EWORKSPACE
    # the attention call on prepared K/V: k and v may be NULL only with the flag; the fused projection itself keeps
    # its one-document restriction, and the entry point without a workspace cannot take prepared K/V at all
    p, a = _qkv_args(); a.k = a.v = 0
    assert lib.pkh3_attn_fwd(C.byref(a), None) == _lib.PKH3_ENULL
    a.flags = _lib.FLAG_KV_PREPARED
    assert lib.pkh3_attn_fwd_noalloc(C.byref(a), None) == _lib.PKH3_EUNSUPPORTED
    a.B = 2
    assert lib.pkh3_qkv_proj(C.byref(p), C.byref(a), None) == _lib.PKH3_EUNSUPPORTED


def test_kv_prepare_argument_errors(lib):
    """The K/V side alone: q and o are not looked at, everything else is checked as in the attention call."""
    a = _valid_args()
    a.q = a.o = 0
    a.k = 0
    assert lib.pkh3_kv_prepare(C.byref(a), None) == _lib.PKH3_ENULL
    a = _valid_args(); a.q = a.o = 0; a.workspace_bytes = 1024
    assert lib.pkh3_kv_prepare(C.byref(a), None) == _lib.PKH3_EWORKSPACE
    a = _valid_args(); a.q = a.o = 0; a.flags = _lib.FLAG_KV_PREPARED
    assert lib.pkh3_kv_prepare(C.byref(a), None) == _lib.PKH3_EARG
    a = _valid_args(); a.q = a.o = 0; a.v_ss = 132
    assert lib.pkh3_kv_prepare(C.byref(a), None) == _lib.PKH3_ESTRIDE
    assert lib.pkh3_kv_prepare(None, None) == _lib.PKH3_ENULL
    # the K/V side of the workspace does not move with the queries or the block map of the later calls
    a = _valid_args()
    dense = lib.pkh3_workspace_bytes(C.byref(a))
    a.Sq = 100000
    assert lib.pkh3_workspace_bytes(C.byref(a)) == dense
    a.blk_row_ptr, a.blk_col_idx = 0x20000, 0x30000
    assert lib.pkh3_workspace_bytes(C.byref(a)) > dense
    # long dense calls: behind the K/V side, a bounded scratch for the workgroup pairs that may end the call
    a = _valid_args(); a.Sk = 4096; a.H = 24
    a.Sq = 384
    small = lib.pkh3_workspace_bytes(C.byref(a))
    a.Sq = 48360
    big = lib.pkh3_workspace_bytes(C.byref(a))
    a.Sq = 1 << 20
    assert 0 < big - small <= 512 * 12 * 17408 + 512 * 48 + 512 and lib.pkh3_workspace_bytes(C.byref(a)) == big


def test_out_proj_argument_errors(lib):
    def ok():
        o = _lib.OutArgs()
        o.o_img, o.S, o.K, o.N = 0x400000, 64, 256, 256
        o.proj.w_img = 0x500000
        o.y, o.y_stride = 0x700000, 256
        return o
    assert lib.pkh3_out_proj(None, None) == _lib.PKH3_ENULL
    for mutate, code in [
        (lambda o: setattr(o, "S", 0), _lib.PKH3_ESHAPE), (lambda o: setattr(o, "K", 40), _lib.PKH3_ESHAPE),
        (lambda o: setattr(o, "N", 100), _lib.PKH3_ESHAPE), (lambda o: setattr(o, "o_img", 0), _lib.PKH3_ENULL),
        (lambda o: setattr(o, "y", 0), _lib.PKH3_ENULL), (lambda o: setattr(o, "y_stride", 128), _lib.PKH3_ESTRIDE),
        (lambda o: (setattr(o, "gate", 0x800000), setattr(o, "gate_stride", 100)), _lib.PKH3_ESTRIDE),
        (lambda o: (setattr(o, "residual", 0x800004), setattr(o, "residual_stride", 256)), _lib.PKH3_ESTRIDE),
        (lambda o: setattr(o.proj, "w_img", 0), _lib.PKH3_ENULL),
        (lambda o: (setattr(o.proj, "lora_a_img", 0x600000), setattr(o.proj, "lora_b_img", 0x600000)), _lib.PKH3_EWORKSPACE),
    ]:
        o = ok()
        mutate(o)
        assert lib.pkh3_out_proj(C.byref(o), None) == code, lib.pkh3_last_error()


def test_projection_struct_layouts_match_header():
    header = open(os.path.join(ROOT, "include", "pkh3_attn.h")).read()
    for name, mirror in (("pkh3_linear", _lib.Linear), ("pkh3_qkv_args", _lib.QkvArgs), ("pkh3_out_args", _lib.OutArgs)):
        body = header[header.index("typedef struct %s {" % name): header.index("} %s;" % name)]
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        names = []
        for decl in body.split("{", 1)[1].split(";"):
            decl = decl.strip()
            if not decl:
                continue
            for part in decl.split(","):
                names.append(re.findall(r"[A-Za-z_][A-Za-z_0-9]*", part)[-1])
        assert names == [f[0] for f in mirror._fields_], name
    assert re.search(r"#define\s+PKH3_LORA_RANK\s+128", header) and _lib.LORA_RANK == 128


def test_projection_front_end_refuses_host_tensors():
    import torch

    from pika_h3_flex_amd import projections as P

    x = torch.zeros((8, 64), dtype=torch.bfloat16)
    for fn in (P.pack_rows, P.pack_weight, P.adaln_modulate):
        with pytest.raises(ValueError, match="device memory"):
            fn(x)
    with pytest.raises(ValueError, match="bfloat16"):
        P.pack_rows(x.float())
    with pytest.raises(ValueError):
        P.packed_bytes(8, 48)
    assert P.packed_bytes(300, 64) == 512 * 64 * 2


def test_fused_front_end_refuses_host_buffers():
    """qkv_attention / out_proj hand raw pointers to kernels: a host buffer must be stopped on the host."""
    import torch

    from pika_h3_flex_amd import projections as P

    S, K, H = 16, 128, 1
    img = torch.zeros(P.packed_bytes(S, K), dtype=torch.uint8)
    lin = P.PackedLinear(torch.zeros(P.packed_bytes(128, K), dtype=torch.uint8), 128, K)
    with pytest.raises(ValueError, match="device memory"):
        P.qkv_attention(img, S, lin, lin, lin, heads=H)
    with pytest.raises(ValueError, match="device memory"):
        P.out_proj(None, lin, o_img=img, rows=S)
    with pytest.raises(ValueError, match="either o or o_img"):
        P.out_proj(None, lin)
    with pytest.raises(ValueError, match="number of rows"):
        P.out_proj(None, lin, o_img=img)


def test_headers_compile_as_c_and_a_c_program_links(tmp_path):
    """The boundary is a C ABI: both headers compile as strict C99, and a C program linked against the library calls
    it (version, the workspace sizing of an invalid call, the error string) without a GPU."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "caller.c"
    src.write_text(
        '#include "pkh3_attn.h"\n'
        '#include "pkh3_attn_bench.h"\n'
        "#include <stdio.h>\n"
        "int main(void) {\n"
        "  pkh3_attn_args a = {0};\n"
        "  int rc = pkh3_attn_fwd(&a, 0);\n"
        '  printf("%d %lu %d %s\\n", pkh3_version(), (unsigned long)pkh3_workspace_bytes(&a), rc, pkh3_strerror(rc));\n'
        "  return 0;\n"
        "}\n")
    libdir = os.path.join(ROOT, "pika-h3-flex_amd")
    exe = tmp_path / "caller"
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"), str(src),
                    "-o", str(exe), "-L", libdir, "-lpkh3attn", f"-Wl,-rpath,{libdir}"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split(None, 3)
    assert int(out[0]) == _lib.load().pkh3_version()
    assert int(out[1]) == 0            # invalid arguments: no size
    assert int(out[2]) < 0 and out[3].strip()
