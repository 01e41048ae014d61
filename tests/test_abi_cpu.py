"""The C ABI as far as it can be exercised without a GPU: the library loads,
exports every symbol include/tracea.h and include/tracea_tuner.h declare, and its host-side logic
(errors, version, ConvParams packing, variant table) behaves as documented."""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

import oracle
from tracea_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    names = set()
    for header in ("tracea.h", "tracea_tuner.h", "tracea_graph.h", "tracea_plan.h", "tracea_ttg.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(tracea_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_every_declared_symbol_is_exported():
    names = _declared_functions()
    assert len(names) >= 20
    handle = C.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), "libtracea.so does not export " + n
    # and the Python binding covers the same set
    assert sorted(capi.SIGNATURES) == names


def test_struct_sizes_match_the_header():
    assert C.sizeof(capi.TensorView) == 40
    assert C.sizeof(capi.Conv2dParams) == 40
    assert C.sizeof(capi.GemmParams) == 16
    assert C.sizeof(capi.AttentionParams) == 24
    assert C.sizeof(capi.ConvParamsBlock) == 80
    assert C.sizeof(capi.Result) == 32


def test_version_is_0_1_0():
    # tracea-ffi/src/lib.rs:244-251
    l = capi.lib()
    assert (l.tracea_version_major(), l.tracea_version_minor(), l.tracea_version_patch()) == (0, 1, 0)


def test_last_error_slot_semantics():
    # tracea-ffi/src/lib.rs:77-109: NUL-terminated, truncated to len-1, -1 for a bad buffer
    l = capi.lib()
    l.tracea_clear_error()
    assert capi.last_error() == ""
    blk = capi.ConvParamsBlock()
    st = l.tracea_conv_params_pack(0, 8, 8, 8, 8, 3, 3, 1, 1, 1, C.byref(blk))
    assert st == capi.INVALID_PARAMS
    msg = capi.last_error()
    assert "positive" in msg
    small = C.create_string_buffer(8)
    n = l.tracea_get_last_error(small, 8)
    assert n == 7 and small.raw[7] == 0 and small.raw[:7].decode() == msg[:7]
    assert l.tracea_get_last_error(None, 16) == -1
    assert l.tracea_get_last_error(small, 0) == -1
    l.tracea_clear_error()
    assert capi.last_error() == ""


def test_compute_before_init_is_unknown_error():
    # src/interface/c_bindings.rs:212: no runtime -> UnknownError.  (On a GPU box another
    # test may already have initialised the library; shut it down for this check.)
    l = capi.lib()
    l.tracea_shutdown()
    shape = (C.c_uint64 * 2)(4, 4)
    buf = (C.c_float * 16)()
    tv = capi.TensorView(C.addressof(buf), 2, shape, None, capi.F32, 0)
    out = capi.TensorView(C.addressof(buf), 2, shape, None, capi.F32, 0)
    st = l.tracea_gemm(tv, tv, None, None, C.byref(out), capi.GemmParams(0, None))
    assert st == capi.UNKNOWN_ERROR
    assert "tracea_init" in capi.last_error()


def test_conv_transpose_before_init_is_unknown_error():
    # src/interface/c_bindings.rs:299: no runtime -> UnknownError, before any view is read
    l = capi.lib()
    l.tracea_shutdown()
    shape = (C.c_uint64 * 4)(1, 4, 4, 8)
    tv = capi.TensorView(None, 4, shape, None, capi.F16, 0)
    st = l.tracea_conv_transpose2d(tv, tv, None, None, C.byref(tv), capi.ConvTranspose2dParams())
    assert st == capi.UNKNOWN_ERROR and "tracea_init" in capi.last_error()
    st = l.tracea_conv_transpose2d_ex(tv, tv, C.byref(tv), capi.ConvTranspose2dParams(), None, 0)
    assert st == capi.UNKNOWN_ERROR


@pytest.mark.parametrize("shape", [
    (32, 56, 56, 64, 64, 3, 3, 1, 1, 1),    # ResNet 3x3 stage (reference preset benchmark.rs:491-493)
    (32, 28, 28, 128, 128, 3, 3, 1, 1, 1),  # basic block
    (32, 56, 56, 64, 128, 3, 3, 2, 1, 1),   # downsampling conv
    (32, 56, 56, 64, 128, 1, 1, 2, 0, 1),   # 1x1 shortcut
    (1, 8, 8, 32, 32, 3, 3, 1, 1, 1),       # examples/verify_conv2d.rs
    (2, 9, 9, 24, 8, 3, 3, 1, 2, 2),
])
def test_conv_params_block_equals_oracle_bit_for_bit(shape):
    blk = capi.ConvParamsBlock()
    st = capi.lib().tracea_conv_params_pack(*shape, C.byref(blk))
    assert st == capi.SUCCESS, capi.last_error()
    ref = oracle.conv_params(*shape)
    assert bytes(blk) == bytes(ref)


def test_variant_table():
    gemm = capi.variants("gemm")
    assert gemm and gemm == capi.variants("conv2d")
    assert all(re.match(r"t\d+x\d+x\d+_w\dx\d", n) or re.match(r"c\d+x\d+_w\dx\d_s\d_patch", n) or
               re.match(r"c\d+x\d+_k\d+_resident", n) or re.match(r"c\d+x\d+_c\d+(_s\d|_r\d|_w\d)?_w16_(resident|patch|ksplit|thin)", n)
               for n in gemm)
    attn = capi.variants("attention")
    assert any("d128" in n for n in attn)
    l = capi.lib()
    assert l.tracea_variant_count(b"nope") == -1
    assert l.tracea_variant_name(b"gemm", 999) is None
    assert l.tracea_force_variant(b"gemm", len(gemm)) == -1
    assert l.tracea_force_variant(b"gemm", 0) == 0
    assert l.tracea_force_variant(b"gemm", -1) == 0


def test_tune_without_runtime_reports_failure():
    l = capi.lib()
    l.tracea_shutdown()
    ok, score, cfg, err = capi.take_result(l.tracea_tune_gemm(256, 256, 256))
    assert not ok and cfg is None and "tracea_init" in err


def test_cpp_header_compiles_and_links(tmp_path):
    """include/tracea.hpp is usable by a plain C++17 caller linked against libtracea.so."""
    import shutil
    import subprocess
    cxx = shutil.which("g++")
    if cxx is None:
        pytest.skip("no g++")
    exe = tmp_path / "hdr"
    libdir = os.path.dirname(capi.LIB_PATH)
    subprocess.check_call([cxx, "-std=c++17", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "cpp_header_check.cpp"), "-o", str(exe),
                           "-L", libdir, "-ltracea", "-Wl,-rpath," + libdir])
    out = subprocess.check_output([str(exe)]).decode()
    assert "tracea.hpp ok" in out


def test_tuner_cli_usage_and_failure_without_a_device(tmp_path):
    """tracea-tuner keeps the reference CLI's sub-commands (src/bin/tuner.rs:11-30) and fails
    cleanly when no device can be initialised."""
    exe = os.path.join(ROOT, "tracea_amd", "bin", "tracea-tuner")
    assert os.path.exists(exe), "run `python -m tracea_amd.build`"
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0 and "gemm <m> <n> <k> [--out <file>]" in r.stderr
    r = subprocess.run([exe, "pool", "1"], capture_output=True, text=True)
    assert r.returncode == 2 and "Unknown subcommand: pool" in r.stderr
    r = subprocess.run([exe, "gemm", "64", "x"], capture_output=True, text=True)
    assert r.returncode == 2
    import torch
    if not torch.cuda.is_available():
        out = tmp_path / "r.json"
        r = subprocess.run([exe, "gemm", "64", "64", "64", "--out", str(out)], capture_output=True, text=True)
        assert r.returncode == 1 and "Runtime init failed" in r.stderr and not out.exists()
