"""The C-ABI boundary and the host-side logic, without a GPU: libscmx.so loads and exports every entry point
include/scmx.h declares (with the argument counts the ctypes table binds), argument checks return their error codes
before anything is launched, and the host helpers that mirror the reference's call surface (e2e/sc_kernels.py:14-27,
471-476; e2e/sc_format.py:26-102; e2e/sc_moe.py:155-166) agree with the numpy oracle."""
import ctypes as C
import importlib.util
import os
import re
import shutil
import subprocess

import numpy as np
import pytest
import torch

from oracle import layout, linear, moe
from tests.conftest import ROOT


@pytest.fixture(scope="module")
def pkg():
    import mxfp4_int8_m5_amd as p
    if not os.path.exists(p._lib.LIB_PATH):        # tests use what is built and build only if nothing is
        import __graft_entry__
        __graft_entry__.build()
    return p


def header_entries():
    text = open(os.path.join(ROOT, "include", "scmx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(scmx_\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args in ("", "void") else args.count(",") + 1
    return out


def test_every_declared_entry_point_is_exported_and_bound(pkg):
    decl = header_entries()
    assert len(decl) >= 24 and {"scmx_mm_w4a8", "scmx_gemv", "scmx_moe_mm", "scmx_quantize_sc"} <= set(decl)
    lib = pkg._lib.load()
    for name, nargs in decl.items():
        assert hasattr(lib, name), f"{name} is declared in include/scmx.h but not exported by libscmx.so"
        assert name in pkg._lib.SIGNATURES, f"{name} has no ctypes binding"
        assert len(pkg._lib.SIGNATURES[name][1]) == nargs, f"{name}: binding has a different number of arguments"
    assert set(pkg._lib.SIGNATURES) == set(decl)


def test_version_default_format_and_workspace_size(pkg):
    lib = pkg._lib.load()
    assert b"gfx950" in lib.scmx_version()
    f = pkg._lib.CFormat()
    lib.scmx_default_format(C.byref(f))
    d = pkg.sc_format.DEFAULT
    assert (f.block, f.bc_bits, f.n_mult) == (d.block, d.bc_bits, len(d.mult))
    assert tuple(f.code_mag) == tuple(d.code_mag) and tuple(f.mult)[:4] == tuple(d.mult)
    for m, k in ((1, 128), (2048, 2048), (77, 6144)):
        mp = (m + 31) // 32 * 32           # whole 32-row blocks of the blocked activation layout
        assert lib.scmx_linear_w4a8_workspace(m, k) == (mp * k + 255) // 256 * 256 + 4 * mp


def test_argument_errors_return_before_any_launch(pkg):
    """Bad shapes, null pointers and unsupported formats are refused with the documented codes and a message; none of
    these calls reaches the device (the pointers below are not device memory)."""
    lib = pkg._lib.load()
    fmt = pkg.sc_format.DEFAULT.c_struct()
    buf = (C.c_char * 4096)()
    p = C.addressof(buf) // 256 * 256 + 256
    assert lib.scmx_mm_w4a8(C.byref(fmt), p, p, p, p, p, None, p, 1, 4, 8, 100, None) == -1          # K % 128
    assert b"K" in lib.scmx_last_error()
    assert lib.scmx_mm_w4a8(C.byref(fmt), None, p, p, p, p, None, p, 1, 4, 8, 128, None) == -1        # null xq
    assert lib.scmx_mm_w4a8(C.byref(fmt), p, p, p, p, p, None, p, 2, 4, 8, 128, None) == -1           # EPI 2 without res
    assert lib.scmx_mm_w4a8(C.byref(fmt), p, p, p, p, p, None, p, 7, 4, 8, 128, None) == -1           # unknown epilogue
    bad = pkg._lib.CFormat()
    C.memmove(C.byref(bad), C.byref(fmt), C.sizeof(bad))
    bad.bc_bits = 3
    assert lib.scmx_mm_w4a8(C.byref(bad), p, p, p, p, p, None, p, 1, 4, 8, 128, None) == -2           # format
    assert lib.scmx_linear_w4a8(C.byref(fmt), p, p, p, p, None, p, 1, 4, 8, 128, p, 16, None) == -4   # workspace
    assert lib.scmx_gemv(C.byref(fmt), p, None, p, p, p, None, p, 1, 1, None, 0.0, 3, 8, 128, None, 0, 0, -1, None) == -1
    assert lib.scmx_quantize_sc(p, 0, 4, 96, 32, p, p, p, None) == -1                                 # K % (4 * block)
    assert lib.scmx_quantize_sc(p, 0, 4, 128, 24, p, p, p, None) == -1                                # block
    assert lib.scmx_attn_decode(p, p, p, None, 5, p, 4, 2, 96, 64, 0.1, None, 1, None) == -1          # head dim
    assert lib.scmx_attn_decode(p, p, p, None, 5, p, 4, 2, 128, 64, 0.1, None, 4, None) == -1         # splits without workspace
    assert lib.scmx_attn_decode_qkv(p, p, p, 1e-6, p, None, 64, p, p, p, 4, 2, 128, 64, 0.1, None, 1, None) == -1  # position outside the cache
    assert lib.scmx_route_sort(p, 4, 8, 2000, 64, p, p, p, p, p, None) == -1                          # experts > 1024
    assert lib.scmx_mm_w4a8(C.byref(fmt), p, p, p, p, p, None, p, 1, 0, 8, 128, None) == 0            # M = 0: nothing to do


def test_mxfp4_in_place_descriptor(pkg):
    """The descriptor of a standard MXFP4 tensor read in place: block 32, one byte per block, no multiplier table; the
    Python Format and the C filler agree; entry points that cannot decode it without row scales say so before any launch."""
    lib = pkg._lib.load()
    F = pkg.sc_format
    c = pkg._lib.CFormat()
    lib.scmx_mxfp4_format(C.byref(c))
    p = F.MXFP4.c_struct()
    assert (c.block, c.bc_bits, c.n_mult) == (32, 8, 0) == (p.block, p.bc_bits, p.n_mult)
    assert list(c.code_mag) == list(p.code_mag) == [0, 1, 2, 3, 4, 6, 8, 12] and not any(c.mult) and not any(p.mult)
    assert F.MXFP4.e8m0 and not F.DEFAULT.e8m0 and F.MXFP4.bits_per_weight(2048) == pytest.approx(4.25 + 32 / 2048)
    buf = (C.c_char * 4096)()
    q = C.addressof(buf) // 256 * 256 + 256
    assert lib.scmx_unpack_i8(C.byref(c), q, q, q, 4, 128, None) == -2 and b"E8M0" in lib.scmx_last_error()
    assert lib.scmx_mm_w4a8(C.byref(c), q, None, q, q, None, None, q, 0, 4, 8, 128, None) == -1      # INT32 out still needs wscale
    assert b"wscale" in lib.scmx_last_error()
    bad = pkg._lib.CFormat()
    C.memmove(C.byref(bad), C.byref(c), C.sizeof(bad))
    bad.code_mag[7] = 10                                                                              # not the E2M1 codebook
    assert lib.scmx_mm_w4a8(C.byref(bad), q, q, q, q, q, None, q, 1, 4, 8, 128, None) == -2
    with pytest.raises(AssertionError):
        F.Format(block=16, mult=(), bc_bits=8)
    with pytest.raises(ValueError):
        pkg.sc_kernels.unpack_i8(None, None, 4, 128, fmt=F.MXFP4)                                     # no row scales given


def test_cpu_tensors_and_missing_library_fail_loudly(pkg, monkeypatch):
    x = torch.zeros((4, 128), dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        pkg.sc_kernels.act_quant(x)                  # a CPU tensor: there is no CPU path
    monkeypatch.setattr(pkg._lib, "_lib", None)
    monkeypatch.setattr(pkg._lib, "LIB_PATH", "/nonexistent/libscmx.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        pkg._lib.load()


def test_host_helpers_match_the_oracle(pkg):
    S, F, M = pkg.sc_kernels, pkg.sc_format, pkg.sc_moe
    assert [S.pad_rows(m) for m in (1, 128, 129, 2048)] == [linear.pad_rows(m) for m in (1, 128, 129, 2048)]
    assert np.array_equal(S.interleave_gate_up(64), linear.interleave_gate_up(64))
    rng = np.random.default_rng(0)
    for ofmt in (layout.Format(), layout.Format(block=16), layout.Format(block=16, mult=(1, 2, 3, 4, 5, 6, 8, 10), bc_bits=4)):
        pf = F.Format(block=ofmt.block, code_mag=tuple(ofmt.code_mag), mult=tuple(ofmt.mult), bc_bits=ofmt.bc_bits)
        c4 = rng.integers(0, 16, (8, 256)).astype(np.uint8)
        b = rng.integers(0, len(ofmt.mult), (8, 256 // ofmt.block)).astype(np.uint8)
        ws = rng.random(8).astype(np.float32)
        for got, want in zip(F.pack_rows(c4, b, ws, pf), layout.pack_rows(c4, b, ws, ofmt)):
            assert got.dtype == want.dtype and np.array_equal(got, want)
        assert np.array_equal(F.decode_numpy(*F.pack_rows(c4, b, ws, pf)[:2], 8, 256, pf),
                              layout.decode(*layout.pack_rows(c4, b, ws, ofmt)[:2], 8, 256, ofmt))
        assert pf.bits_per_weight(4096) == pytest.approx(4 + ofmt.bc_bits / ofmt.block + 32 / 4096)
    with pytest.raises(AssertionError):
        F.Format(block=12)
    with pytest.raises(AssertionError):
        F.Format(code_mag=(0, 1, 2, 3, 4, 6, 8, 12), mult=(1, 2, 4, 16))      # 12 * 16 does not fit INT8
    es = np.sort(rng.integers(0, 8, 300)).astype(np.int32)
    es[es == 5] = 6                                                           # an empty expert
    off, ts, mt = M.segments(torch.from_numpy(np.sort(es)), 8, 64)
    ro = moe.route_sort(np.sort(es).reshape(-1, 1), 8, 64)
    assert np.array_equal(off.numpy(), ro[3]) and np.array_equal(ts.numpy(), ro[4]) and mt == -(-300 // 64) + 8


def test_attention_split_policy_and_cache_names(pkg):
    """Host-side choices that never touch the GPU: row ranges of the decode attention by context length, and the
    packed-cache file names of the reference (e2e/pack_format.py:79-80, e2e/fused_qwen3.py:331-333)."""
    S = pkg.sc_kernels
    assert [S.attn_splits(n) for n in (1, 512, 1024, 1025, 4096, 100000)] == [1, 1, 1, 8, 8, 16]
    from mxfp4_int8_m5_amd import pack_format as PF
    assert PF.cache_path("Qwen/Qwen3-1.7B", "e2m1/B16/M1..10", "/c") == "/c/Qwen--Qwen3-1.7B-fmt-e2m1_B16_M110.safetensors"
    f = PF.sc_format_of("e2m1/B16/M1..10")
    assert (f.block, f.bc_bits, tuple(f.mult)) == (16, 4, tuple(range(1, 11)))
    f = PF.sc_format_of("e2m1/B32/pow2")
    assert (f.block, f.bc_bits, tuple(f.mult)) == (32, 2, (1, 2, 4, 8))
    # row tile of the grouped GEMM by rows per expert (64 experts: 512 tokens x 8 -> 64 rows each, 1024 -> 128)
    assert [pkg.sc_moe.row_tile(t * 8, 64) for t in (1, 512, 767, 768, 4096)] == [64, 64, 64, 256, 256]


@pytest.mark.skipif(shutil.which(os.environ.get("HIPCC", "hipcc")) is None, reason="needs hipcc to build the instrumented library")
def test_host_code_under_address_and_undefined_behaviour_sanitizers():
    """The library's host code (argument checks, launch-shape arithmetic, dispatch) compiled with AddressSanitizer and
    UBSan and driven by tests/boundary_driver.cpp on this machine, which has no GPU: every entry point with null
    pointers, bad shapes and formats, plausible arguments (which end at the failing launch) and 4000 rounds of seeded
    random integers including the 32-bit extremes.  A sanitizer report aborts the driver; a wrong status makes it
    exit 1.  Exit 77 = a GPU is present (the driver passes addresses that are not memory), which skips the test."""
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    spec = importlib.util.spec_from_file_location("scmx_build", os.path.join(ROOT, "mxfp4-int8-m5_amd", "build.py"))
    builder = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(builder)
    exe = builder.build_host_check(os.path.join(ROOT, "tests", "boundary_driver.cpp"))
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600, env=env)
    if run.returncode == 77:
        pytest.skip("a GPU is present")
    assert run.returncode == 0, run.stdout[-4000:]
    assert "0 failure(s)" in run.stdout and "runtime error" not in run.stdout and "AddressSanitizer" not in run.stdout
