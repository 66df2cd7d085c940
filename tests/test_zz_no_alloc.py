"""The dense layer's entry point that allocates nothing (scmx_linear_w4a8_static: the INT8 activations and their scales
live in a fixed array of the library's device image) against scmx_linear_w4a8 with a caller workspace, through the C
ABI: bit-identical outputs on two calls in a row, the second with a smaller input, every epilogue; sizes beyond the
built-in scratch are refused."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import bf16, linear
from tests.util import dev, host, llm_acts, random_packed

pytestmark = pytest.mark.gpu
F32 = np.float32


def _call(lib, name, *args):
    rc = getattr(lib, name)(*args)
    return rc, lib.scmx_last_error().decode()


def test_static_scratch_entry_point_equals_the_workspace_one():
    from mxfp4_int8_m5_amd import _lib, sc_format
    lib = _lib.load()
    fmt = sc_format.DEFAULT.c_struct()
    sp = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(77)
    # first call large (fills most of a 2048 x 2048 slice of the scratch), second smaller with other K: what the first
    # call left in the array must not show in the second
    for (m, n, k, epi) in [(2048, 512, 2048, 1), (300, 384, 1024, 2), (37, 256, 128, 3), (1, 64, 6144, 1)]:
        codes, bc, ws, q = random_packed(rng, n, k)
        bits, x = llm_acts(rng, m, k)
        res = bf16.to_bits(rng.standard_normal((m, n)).astype(F32))
        dx, dc, db, dw, dr = dev(bits), dev(codes), dev(bc), dev(ws), dev(res)
        no = n // 2 if epi == 3 else n
        out_a = torch.zeros((m, no), dtype=torch.bfloat16, device="cuda")
        out_b = torch.zeros((m, no), dtype=torch.bfloat16, device="cuda")
        need = lib.scmx_linear_w4a8_workspace(m, k)
        wsp = torch.empty(need, dtype=torch.uint8, device="cuda")
        rp = dr.data_ptr() if epi == 2 else None
        rc, msg = _call(lib, "scmx_linear_w4a8", C.byref(fmt), dx.data_ptr(), dc.data_ptr(), db.data_ptr(), dw.data_ptr(),
                        rp, out_a.data_ptr(), epi, m, n, k, wsp.data_ptr(), need, sp)
        assert rc == 0, msg
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        rc, msg = _call(lib, "scmx_linear_w4a8_static", C.byref(fmt), dx.data_ptr(), dc.data_ptr(), db.data_ptr(),
                        dw.data_ptr(), rp, out_b.data_ptr(), epi, m, n, k, sp)
        assert rc == 0, msg
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(out_a, out_b), (m, n, k, epi)
        # and both are the oracle's layer
        xq, xs = linear.act_quant(x)
        ref = linear.epilogue(linear.int_gemm(xq, q), xs, ws, epi, res if epi == 2 else None)
        assert np.array_equal(host(out_b), ref), (m, n, k, epi)


def test_static_scratch_limits_are_refused():
    from mxfp4_int8_m5_amd import _lib, sc_format
    lib = _lib.load()
    fmt = sc_format.DEFAULT.c_struct()
    sp = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.scmx_linear_w4a8_static_max_elements() == 16 * 2 ** 20 and lib.scmx_linear_w4a8_static_max_rows() == 16384
    t = torch.zeros(64, dtype=torch.uint8, device="cuda")     # never touched: the call must fail before any launch
    p = t.data_ptr()
    for m, k in ((8192, 2176), (16385, 128)):
        rc, msg = _call(lib, "scmx_linear_w4a8_static", C.byref(fmt), p, p, p, p, None, p, 1, m, 128, k, sp)
        assert rc == -4 and "beyond the built-in scratch" in msg
    rc, msg = _call(lib, "scmx_linear_w4a8_static", C.byref(fmt), p, p, p, p, None, p, 1, -1, 128, 128, sp)
    assert rc == -1
