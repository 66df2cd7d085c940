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
    # call left in the array must not show in the second.  The 4096-wide case is large enough for the blocked activation
    # layout (ragged M: the last 32-row block is partly padding); the narrow ones quantize by rows into the same array.
    shapes = [(2048, 512, 2048, 1), (2047, 4096, 1024, 2), (300, 384, 1024, 2), (37, 256, 128, 3), (1, 64, 6144, 1)]
    assert lib.scmx_mm_w4a8_prefers_blocked(2047, 4096, 1024) == 1 and lib.scmx_mm_w4a8_prefers_blocked(300, 384, 1024) == 0
    for (m, n, k, epi) in shapes:
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
        assert lib.scmx_init() == 0          # address look-ups done: nothing below may change the device's free memory
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        rc, msg = _call(lib, "scmx_linear_w4a8_static", C.byref(fmt), dx.data_ptr(), dc.data_ptr(), db.data_ptr(),
                        dw.data_ptr(), rp, out_b.data_ptr(), epi, m, n, k, sp)
        assert rc == 0, msg
        torch.cuda.synchronize()
        # torch's counter sees only torch's allocator; the driver's free-memory figure sees a hipMalloc by anyone
        assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
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


def test_static_entry_point_inside_a_captured_graph():
    """The use the entry point is meant for: after scmx_init() on the device, the call is captured into a HIP graph and
    replayed with changed inputs; every replay equals the eager workspace entry point."""
    from mxfp4_int8_m5_amd import _lib, sc_format
    lib = _lib.load()
    fmt = sc_format.DEFAULT.c_struct()
    assert lib.scmx_init() == 0
    rng = np.random.default_rng(78)
    m, n, k = 192, 512, 1024
    codes, bc, ws, q = random_packed(rng, n, k)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    x = torch.zeros((m, k), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((m, n // 2), dtype=torch.bfloat16, device="cuda")       # SwiGLU: the epilogue that reads the table
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        sp = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc, msg = _call(lib, "scmx_linear_w4a8_static", C.byref(fmt), x.data_ptr(), dc.data_ptr(), db.data_ptr(),
                        dw.data_ptr(), None, y.data_ptr(), 3, m, n, k, sp)
        assert rc == 0, msg
    torch.cuda.current_stream().wait_stream(side)
    need = lib.scmx_linear_w4a8_workspace(m, k)
    wsp = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = torch.zeros_like(y)
    sp0 = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for seed in (1, 2, 3):
        bits, xf = llm_acts(np.random.default_rng(seed), m, k)
        x.copy_(dev(bits))
        graph.replay()
        rc, msg = _call(lib, "scmx_linear_w4a8", C.byref(fmt), x.data_ptr(), dc.data_ptr(), db.data_ptr(), dw.data_ptr(),
                        None, want.data_ptr(), 3, m, n, k, wsp.data_ptr(), need, sp0)
        assert rc == 0, msg
        torch.cuda.synchronize()
        assert torch.equal(y, want), seed
        xq, xs = linear.act_quant(xf)
        with np.errstate(all="ignore"):
            assert np.array_equal(host(y), linear.epilogue(linear.int_gemm(xq, q), xs, ws, 3)), seed
