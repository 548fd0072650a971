"""The C-ABI library loads, exports every symbol include/dtas_abi.h declares, and its host-side
logic (bucket selection, argument checks, error reporting) behaves -- no kernel is launched here."""
import ctypes
import os
import re

import pytest

from dtas_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = open(os.path.join(ROOT, "include", "dtas_abi.h")).read()


def declared_functions():
    body = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    return sorted(set(re.findall(r"\b(dtas_\w+)\s*\(", body)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 19
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(handle, name), f"{name} is declared in dtas_abi.h but not exported"
    # and the Python binding knows each of them
    assert set(names) == set(_lib.SIGNATURES) | {"dtas_last_error"}


def test_abi_version_and_struct_layout():
    assert _lib.lib().dtas_abi_version() == _lib.ABI_VERSION
    assert ctypes.sizeof(_lib.DtasConfig) == 40          # 8 x int32 + int64
    assert ctypes.sizeof(_lib.DtasLaunchInfo) == 7 * 8 + 16 + 8 + 40 + 96


def test_select_bucket_uses_labelled_ranges():
    # built-in tables: bucket width 16 up to 8192; n = 16 belongs to [1, 16], n = 17 to [17, 32]
    a = _lib.select_bucket(_lib.OP_GEMM_F16, 16, 4096, 4096)
    b = _lib.select_bucket(_lib.OP_GEMM_F16, 17, 4096, 4096)
    assert (a.index, b.index) == (0, 1)
    assert a.name == b"fused_NT_matmul4_add1_n_1_to_16__kernel"
    # 16 rows against 4096 x 4096: the W-streaming kernel, 64 columns x 1024 of K per workgroup, one workgroup per CU
    assert a.config.variant == _lib.GEMM_STREAM and list(a.config.tile) == [16, 64, 1024]
    assert list(a.launch_args)[:5] == [256, 1, 1, 256, (16 + 64) * 1024 * 2]
    wide = _lib.select_bucket(_lib.OP_GEMM_F16, 16, 32000, 4096)   # more workgroups than CUs: the tiles
    assert wide.config.variant == _lib.GEMM_MFMA
    big = _lib.select_bucket(_lib.OP_GEMM_F16, 4096, 4096, 4096)
    assert big.config.variant == _lib.GEMM_MFMA and list(big.config.tile) == [256, 256, 64]
    assert list(big.launch_args)[:4] == [256, 1, 1, 512] and big.launch_args[4] == 5 * 256 * 128  # a ring of five operand units
    assert big.bucket_lo <= 4096 <= big.bucket_hi
    # extents above the upper bound share the last bucket
    assert _lib.select_bucket(_lib.OP_GEMM_F16, 100000, 4096, 4096).index == 511


def test_select_bucket_table_rows_are_monotone_and_merged():
    rows, last = [], None
    for n in range(1, 8193, 16):
        info = _lib.select_bucket(_lib.OP_RMS_NORM_F16, n, 4096, 0)
        assert info.bucket_lo <= n <= info.bucket_hi
        rows.append(info.table_row)
        if last is not None and info.table_row == last.table_row:
            assert info.config.to_dict() == last.config.to_dict()
        last = info
    assert rows == sorted(rows) and rows[0] == 0 and rows[-1] == len(set(rows)) - 1


def test_elementwise_launch_shape():
    info = _lib.select_bucket(_lib.OP_ADD_F16, 4096, 4096, 0)
    c = info.config
    assert (c.variant, c.block, c.vec) == (_lib.ELT_VECTOR, 256, 8)
    assert info.launch_args[0] == -(-(4096 * 4096 // 8) // (256 * c.unroll)) and info.launch_args[3] == 256
    assert _lib.select_bucket(_lib.OP_ADD_I8, 1, 2560, 0).config.vec == 16
    assert _lib.select_bucket(_lib.OP_ADD_F32, 1, 2560, 0).config.vec == 4
    # a cast moves 128 bit on the wider side: 4 elements per access in either direction
    assert _lib.select_bucket(_lib.OP_CAST_F32_F16, 1, 4096, 0).config.vec == 4
    assert _lib.select_bucket(_lib.OP_CAST_F16_F32, 1, 4096, 0).config.vec == 4
    # accesses in flight per thread shrink with the extent so that the grid still fills the CUs
    assert [_lib.select_bucket(_lib.OP_ADD_F16, n, 4096, 0).config.unroll for n in (1, 128, 1024, 4096)] == [1, 1, 2, 8]


def test_describe_launch_rejects_bad_configs():
    cfg = _lib.DtasConfig.from_dict({"variant": 0, "block": 128, "vec": 8, "unroll": 4})
    with pytest.raises(_lib.DtasError, match="block must be 256"):
        _lib.describe_launch(_lib.OP_ADD_F16, 16, 4096, 0, cfg)
    cfg = _lib.DtasConfig.from_dict({"variant": 0, "block": 256, "vec": 3, "unroll": 4})
    with pytest.raises(_lib.DtasError, match="vector width"):
        _lib.describe_launch(_lib.OP_ADD_F16, 16, 4096, 0, cfg)
    cfg = _lib.DtasConfig.from_dict({"variant": 0, "block": 256, "vec": 8, "unroll": 1, "tile": [100, 100, 64]})
    with pytest.raises(_lib.DtasError, match="no MFMA kernel"):
        _lib.describe_launch(_lib.OP_GEMM_F16, 512, 4096, 4096, cfg)
    # a wavefront cannot hold a 100k-element row in registers
    cfg = _lib.DtasConfig.from_dict({"variant": _lib.RED_WAVE_ROW, "block": 256, "vec": 8, "unroll": 1})
    with pytest.raises(_lib.DtasError, match="does not fit"):
        _lib.describe_launch(_lib.OP_RMS_NORM_F16, 4, 100000, 0, cfg)


def _call(name, *args):
    return getattr(_lib.lib(), name)(*args)


def test_argument_errors_return_minus_one_with_a_message():
    fake_a, fake_b, fake_c = 0x10000, 0x20000000, 0x40000000   # never dereferenced: every call fails first
    assert _call("dtas_add_f16", fake_a, fake_b, fake_c, -1, 4096, None, None) == -1
    assert "negative extent" in _lib.last_error()
    assert _call("dtas_add_f16", None, fake_b, fake_c, 4, 4096, None, None) == -1
    assert "NULL buffer" in _lib.last_error()
    assert _call("dtas_add_f16", fake_a, fake_b, fake_a + 64, 4, 4096, None, None) == -1
    assert "overlaps" in _lib.last_error()
    assert _call("dtas_gemm_f16", fake_a, fake_b, None, fake_c, 4, -2, 64, None, None) == -1
    assert _call("dtas_softmax_f16", fake_a, fake_a, 4, 128, None, None) == -1
    assert "overlaps" in _lib.last_error()
    assert _call("dtas_select_bucket", 99, 1, 1, 1, ctypes.byref(_lib.DtasLaunchInfo())) == -1
    assert "unknown op" in _lib.last_error()


def test_attn_scores_with_an_empty_head_dimension_fails_before_any_division():
    # d = 0 passes the d % 8 check; the row kernel's launch shape divides by d / 8, so it must be refused first
    fake_q, fake_k, fake_m, fake_o = 0x10000, 0x20000000, 0x30000000, 0x40000000   # never dereferenced
    cfg = _lib.DtasConfig.from_dict({"variant": _lib.GEMM_SKINNY, "block": 1024, "vec": 8, "unroll": 1, "tile": [1, 8, 0], "split_k": 1})
    assert _call("dtas_attn_scores_f16_f32", fake_q, fake_k, fake_m, fake_o, 1, 1, 8, 0, 0.1, ctypes.byref(cfg), None) == -1
    assert "head dimensions from 8" in _lib.last_error()


def test_empty_extent_is_a_successful_no_op():
    assert _call("dtas_add_f16", None, None, None, 0, 4096, None, None) == 0
    assert _lib.last_error() == ""            # a success clears the previous message
    assert _call("dtas_rms_norm_f16", None, None, None, 0, 4096, 1e-5, None, None) == 0
    assert _call("dtas_softmax_f16", None, None, 0, 0, None, None) == 0
    assert _call("dtas_gemv_f16", None, None, None, None, 0, 4096, None, None) == 0
    assert _call("dtas_gemv_f16_fused", None, None, None, None, None, None, 0, 4096, 3, None, None) == 0
    assert _call("dtas_gemv_f16_fused", None, None, None, None, None, None, 0, 4096, 9, None, None) == -1
    assert _call("dtas_gemm_f16", None, None, None, None, 0, 4096, 4096, None, None) == 0


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libdtas_gfx950.so")
    with pytest.raises(ImportError, match="no fallback"):
        _lib.lib()


def test_header_is_plain_c_and_a_c_caller_links(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 (no C++ in it), and a C program that calls an
    entry point through it must link against the library (no GPU needed: the call fails its argument check)."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None or not os.path.exists(_lib.LIB_PATH):
        pytest.skip("needs gcc and the built library")
    src = tmp_path / "caller.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "dtas_abi.h"\n'
        "int main(void) {\n"
        "  struct dtas_config cfg; memset(&cfg, 0, sizeof cfg);\n"
        "  if (dtas_abi_version() != DTAS_ABI_VERSION) return 1;\n"
        "  if (dtas_add_f16(NULL, NULL, NULL, -1, 8, NULL, NULL) != -1) return 2;   /* negative extent */\n"
        '  if (strstr(dtas_last_error(), "negative") == NULL) return 3;\n'
        "  if (dtas_gemv_q8_f16(NULL, NULL, NULL, NULL, NULL, 4, 48, DTAS_EPI_BIAS, NULL, NULL) != -1) return 4;\n"
        "  if (dtas_attn_pv_f16(NULL, NULL, NULL, 0, 0, 0, 80, NULL, NULL) != 0) return 5;     /* empty: no-op */\n"
        '  puts("ok");\n  return 0;\n}\n')
    include = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    libdir = os.path.dirname(_lib.LIB_PATH)
    exe = tmp_path / "caller"
    subprocess.check_call([gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", include, str(src), "-o", str(exe),
                           "-L", libdir, "-ldtas_gfx950", f"-Wl,-rpath,{libdir}"])
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "ok", (out.returncode, out.stdout, out.stderr)
