"""Dense prefill parity on the GPU, through the C ABI: unpack, activation quantization, INT32 GEMM (bit-exact) and
the scaling epilogues, against the numpy oracle.  Mirrors e2e/test_sc_kernels.py:33-51,121-157 and
e2e/test_formats.py:26-36 of the reference."""
import numpy as np
import pytest
import torch

from oracle import bf16, layout, linear
from tests.util import FORMATS, blocked_layout, dev, host, llm_acts, llm_weights, product_format, random_packed

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def S():
    from mxfp4_int8_m5_amd import sc_kernels
    yield sc_kernels
    sc_kernels.set_format(product_format(layout.DEFAULT))


def test_unpack_quantized_matrix(S):
    rng = np.random.default_rng(0)
    n, k = 384, 2048
    w = rng.standard_normal((n, k)) * 0.02 * rng.lognormal(0, 0.3, (1, k))
    codes, bc, ws, qw = layout.quantize(w)
    wq = host(S.unpack_i8(dev(codes), dev(bc), n, k, lazy=False))
    assert np.array_equal(wq, qw)
    assert np.array_equal(wq, layout.decode(codes, bc, n, k))


@pytest.mark.parametrize("i", range(len(FORMATS)))
def test_unpack_all_formats_random_codes(S, i):
    fmt = FORMATS[i]
    rng = np.random.default_rng(10 + i)
    for n, k in ((256, 2048), (5, 128), (3, 64 if fmt.block * fmt.per_byte <= 64 else 128)):
        if (k // fmt.block) % fmt.per_byte:
            continue
        codes, bc, ws, q = random_packed(rng, n, k, fmt)
        wq = host(S.unpack_i8(dev(codes), dev(bc), n, k, lazy=False, fmt=product_format(fmt)))
        assert np.array_equal(wq, q), (fmt, n, k)


@pytest.mark.parametrize("m,k", [(200, 2048), (1, 128), (130, 6144), (7, 1000)])
def test_act_quant(S, m, k):
    rng = np.random.default_rng(m)
    bits, x = llm_acts(rng, m, k)
    if m > 3:
        bits[3] = 0
        x[3] = 0
    xq, xs = S.act_quant(dev(bits))
    rq, rs = linear.act_quant(x, S.pad_rows(m))
    assert xq.shape[0] == S.pad_rows(m)
    assert np.array_equal(host(xq), rq) and np.array_equal(host(xs), rs)
    assert not host(xq)[m:].any() and not host(xs)[m:].any()


@pytest.mark.parametrize("m,n,k", [(256, 384, 2048), (200, 384, 2048), (512, 2048, 1024), (64, 64, 128), (1, 4, 128),
                                   (1024, 512, 256), (300, 260, 384)])
def test_int32_gemm_exact(S, m, n, k):
    rng = np.random.default_rng(m + n + k)
    codes, bc, ws, q = random_packed(rng, n, k)
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    xq[0] = 127
    ref = linear.int_gemm(xq, q)
    a1 = host(S.mm_i8_i32(dev(xq), dev(q)))
    assert np.array_equal(a1, ref), "INT8-weights GEMM"
    packed = S.unpack_i8(dev(codes), dev(bc), n, k, lazy=True)
    a2 = host(S.mm_i8_i32(dev(xq), packed))
    assert np.array_equal(a2, ref), "fused-unpack GEMM"


@pytest.mark.parametrize("i", range(1, len(FORMATS)))
def test_int32_gemm_other_formats(S, i):
    fmt = FORMATS[i]
    rng = np.random.default_rng(40 + i)
    m, n, k = 128, 256, 2048
    codes, bc, ws, q = random_packed(rng, n, k, fmt)
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    S.set_format(product_format(fmt))
    acc = host(S.mm_i8_i32(dev(xq), S.unpack_i8(dev(codes), dev(bc), n, k)))
    S.set_format(product_format(layout.DEFAULT))
    assert np.array_equal(acc, linear.int_gemm(xq, q))


@pytest.mark.parametrize("m,n,k", [(256, 512, 1024), (128, 256, 2048), (2048, 2048, 256), (200, 136, 128)])
@pytest.mark.parametrize("packed", [False, True])
def test_epilogues(S, m, n, k, packed):
    """EPI 1/2/3 equal the INT32 GEMM + the reference formulas bit for bit (e2e/test_sc_kernels.py:121-142)."""
    rng = np.random.default_rng(m * 7 + n)
    codes, bc, _, q = random_packed(rng, n, k)
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    xs = (np.abs(rng.standard_normal(m)) * 1e-3).astype(F32)
    ws = (np.abs(rng.standard_normal(n)) * 1e-4).astype(F32)
    res = bf16.to_bits(rng.standard_normal((m, n)).astype(F32))
    acc = linear.int_gemm(xq, q)
    wq = S.unpack_i8(dev(codes), dev(bc), n, k, lazy=packed)
    y1 = host(S.mm_epi(dev(xq), wq, dev(xs), dev(ws), 1, torch.bfloat16))
    assert np.array_equal(y1, linear.epilogue(acc, xs, ws, 1))
    y2 = host(S.mm_epi(dev(xq), wq, dev(xs), dev(ws), 2, torch.bfloat16, res=dev(res)))
    assert np.array_equal(y2, linear.epilogue(acc, xs, ws, 2, res))
    perm = linear.interleave_gate_up(n // 2)
    assert np.array_equal(perm, S.interleave_gate_up(n // 2))
    if packed:
        wq3 = S.unpack_i8(dev(codes.reshape(n, -1)[perm].reshape(-1)), dev(bc[perm]), n, k, lazy=True)
    else:
        wq3 = dev(q[perm])
    y3 = host(S.mm_epi(dev(xq), wq3, dev(xs), dev(ws[perm]), 3, torch.bfloat16))
    y = linear.scale_out(acc, xs, ws)
    assert np.array_equal(y3, linear.swiglu(y[:, :n // 2], y[:, n // 2:]))


def test_config0_dense_layer(S):
    """BASELINE config 0: N = K = 2048, M = 512, SC-MXFP4-quantized N(0, 0.02) weights with outlier columns, bf16
    activations with outlier channels; INT32 accumulators bit-exact, bf16 output within 1e-2 of the float path."""
    rng = np.random.default_rng(0)
    n = k = 2048
    m = 512
    w = llm_weights(rng, n, k)
    codes, bc, ws, q = layout.quantize(w)
    bits, x = llm_acts(rng, m, k)
    xq_ref, xs_ref = linear.act_quant(x)
    acc_ref = linear.int_gemm(xq_ref, q)
    xq, xs = S.act_quant(dev(bits), Mp=m)
    assert np.array_equal(host(xq), xq_ref) and np.array_equal(host(xs), xs_ref)
    wq = S.unpack_i8(dev(codes), dev(bc), n, k)
    assert np.array_equal(host(S.mm_i8_i32(xq, wq)), acc_ref)
    y = host(S.linear_w4a8(dev(bits), dev(codes), dev(bc), dev(ws), n))
    assert np.array_equal(y, linear.epilogue(acc_ref, xs_ref, ws, 1))
    ref = linear.float_reference(x, q, ws)
    assert linear.rel_fro(bf16.from_bits(y), ref) < 1e-2          # tolerance stated by the north star
    assert linear.rel_fro(bf16.from_bits(y), x.astype(np.float64) @ w.T) < 0.2   # and it is the layer it claims to be


@pytest.mark.parametrize("name,n,k", [("qkv", 4096, 2048), ("o_proj", 2048, 2048), ("gate_up", 12288, 2048),
                                      ("down", 2048, 6144)])
def test_config1_full_size_m2048(S, name, n, k):
    """BASELINE config 1 at M = 2048: all INT32 accumulators against the float64 integer GEMM, the bf16 epilogue
    bit for bit, and column-linearity of the accumulators (acc(x1 + x2) = acc(x1) + acc(x2))."""
    rng = np.random.default_rng(n + k)
    m = 2048
    codes, bc, ws, q = random_packed(rng, n, k)
    bits, x = llm_acts(rng, m, k)
    xq_ref, xs_ref = linear.act_quant(x)
    acc_ref = linear.int_gemm(xq_ref, q)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    xq, xs = S.act_quant(dev(bits), Mp=m)
    wq = S.unpack_i8(dc, db, n, k)
    acc = host(S.mm_i8_i32(xq, wq))
    assert np.array_equal(acc, acc_ref)
    y = host(S.linear_w4a8(dev(bits), dc, db, dw, n))
    assert np.array_equal(y, linear.epilogue(acc_ref, xs_ref, ws, 1))
    a = rng.integers(-60, 61, (256, k)).astype(np.int8)
    b = rng.integers(-60, 61, (256, k)).astype(np.int8)
    s = host(S.mm_i8_i32(dev(a), wq)) + host(S.mm_i8_i32(dev(b), wq))
    assert np.array_equal(host(S.mm_i8_i32(dev((a + b).astype(np.int8)), wq)), s)


@pytest.mark.parametrize("name,n,k", [("qkv", 4096, 2048), ("o_proj", 2048, 2048), ("gate_up", 12288, 2048),
                                      ("down", 2048, 6144)])
def test_config1_quantized_weights_m2048(S, name, n, k):
    """BASELINE config 1 at M = 2048 with weights generated as config 0 prescribes: N(0, 0.02) with 0.5 % of the input
    columns scaled by 8, spread-constrained SC-MXFP4 quantization (the oracle's restatement of sim/make_testcase.py:
    26-44), activations N(0, 1) with 1 % of the channels scaled by 20.  The one-call layer (quantization prologue +
    fused-unpack GEMM + epilogue) bit for bit against the oracle, and within the north star's 1e-2 relative Frobenius
    error of the float path (sim/make_testcase.py:59-60)."""
    rng = np.random.default_rng(1000 + n + k)
    m = 2048
    w = llm_weights(rng, n, k)
    codes, bc, ws, q = layout.quantize(w)
    assert np.abs(q).max() <= 96
    bits, x = llm_acts(rng, m, k)
    xq_ref, xs_ref = linear.act_quant(x)
    acc_ref = linear.int_gemm(xq_ref, q)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    y = host(S.linear_w4a8(dev(bits), dc, db, dw, n))
    assert np.array_equal(y, linear.epilogue(acc_ref, xs_ref, ws, 1))
    xq, xs = S.act_quant(dev(bits), Mp=m)
    assert np.array_equal(host(S.mm_i8_i32(xq, S.unpack_i8(dc, db, n, k))), acc_ref)
    assert linear.rel_fro(bf16.from_bits(y), linear.float_reference(x, q, ws)) < 1e-2   # the north star's tolerance
    assert linear.rel_fro(bf16.from_bits(y), x.astype(np.float64) @ w.T) < 0.2


def test_bad_arguments_raise(S):
    xq = torch.zeros((4, 100), dtype=torch.int8, device="cuda")
    wq = torch.zeros((8, 100), dtype=torch.int8, device="cuda")
    with pytest.raises(ValueError):
        S.mm_i8_i32(xq, wq)                      # K not a multiple of 128
    with pytest.raises(ValueError):
        S.act_quant(torch.zeros((4, 64), dtype=torch.bfloat16))   # CPU tensor


@pytest.mark.parametrize("m,n,k", [(1, 128, 256), (37, 64, 384), (300, 1024, 512), (700, 2048, 1152), (1100, 12288, 640),
                                   (2047, 4096, 1024)])
def test_linear_one_call(S, m, n, k):
    """linear_w4a8 (quantization prologue + GEMM behind one C entry point): ragged row counts, few and many column
    tiles, a caller-provided workspace that ends up holding the INT8 rows and their scales."""
    rng = np.random.default_rng(m + n + k)
    codes, bc, ws, q = random_packed(rng, n, k)
    bits, x = llm_acts(rng, m, k)
    xq_ref, xs_ref = linear.act_quant(x)
    y_ref = linear.epilogue(linear.int_gemm(xq_ref, q), xs_ref, ws, 1)
    work = torch.full((S.linear_w4a8_workspace(m, k),), 0x55, dtype=torch.uint8, device="cuda")
    y = host(S.linear_w4a8(dev(bits), dev(codes), dev(bc), dev(ws), n, workspace=work))
    assert np.array_equal(y, y_ref)
    wh = host(work)
    mp = (m + 31) // 32 * 32                 # the workspace is laid out for whole 32-row blocks
    by_rows = wh[:m * k].view(np.int8).reshape(m, k)
    padded = np.zeros((mp, k), np.int8)
    padded[:m] = xq_ref
    in_blocks = wh[:mp * k].view(np.int8)    # large shapes are quantized into the blocked layout
    assert np.array_equal(by_rows, xq_ref) or np.array_equal(in_blocks, blocked_layout(padded))
    off = (mp * k + 255) & ~255
    assert np.array_equal(wh[off:off + 4 * m].view(np.float32), xs_ref)


def test_swiglu_epilogue_every_gate_value(S):
    """The SwiGLU epilogue looks silu(g) up in a 65536-entry table built at compile time.  Drive every bf16 bit
    pattern through it as the gate (acc = +-1, xscale = 1, wscale = the value itself) with two different up values
    and compare with the oracle's operation-by-operation bf16 evaluation: bit-exact for every finite gate, NaN where
    the oracle gives NaN."""
    allb = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    gate = bf16.from_bits(allb)                                   # float32 values incl. inf / NaN / denormals
    n, k = 4 * 32768, 128
    ws = np.empty(n, F32)
    ws4 = ws.reshape(-1, 4)
    ws4[:, 0], ws4[:, 1] = gate[0::2], gate[1::2]
    ws4[:, 2], ws4[:, 3] = F32(1.0), F32(-0.3984375)              # up values (bf16-representable)
    code4 = np.zeros((n, k), np.uint8)
    code4[:, 0] = 1                                               # weight row = (1, 0, 0, ...): acc = xq[:, 0]
    codes, bc, _ = layout.pack_rows(code4, np.zeros((n, k // 32), np.uint8), ws)
    xq = np.zeros((2, k), np.int8)
    xq[0, 0], xq[1, 0] = 1, -1
    xs = np.ones(2, F32)
    wq = S.unpack_i8(dev(codes), dev(bc), n, k)
    got = host(S.mm_epi(dev(xq), wq, dev(xs), dev(ws), 3))
    acc = np.stack([np.ones(n, np.int32), -np.ones(n, np.int32)])
    with np.errstate(all="ignore"):
        want = linear.epilogue(acc, xs, ws, 3)
    assert got.shape == want.shape == (2, n // 2)
    nan = np.isnan(bf16.from_bits(want))
    assert np.array_equal(np.isnan(bf16.from_bits(got)), nan)
    assert np.array_equal(got[~nan], want[~nan])
    assert (~nan).sum() > 2 * 65000


@pytest.mark.parametrize("n,k,m", [(384, 1024, 200), (4096, 1024, 2047)])   # the second quantizes into the blocked layout
def test_linear_layer_replays_in_a_hip_graph(S, n, k, m):
    """The entry points only enqueue kernels on the given stream (no allocation, no synchronisation, no memset), so a
    dense layer can be captured once and replayed: every replay, with new activations copied into the captured input
    and eager work in between, equals the eager result bit for bit."""
    rng = np.random.default_rng(21)
    codes, bc, ws, _ = random_packed(rng, n, k)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    x = torch.zeros((m, k), dtype=torch.bfloat16, device="cuda")
    work = torch.empty(S.linear_w4a8_workspace(m, k), dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        S.linear_w4a8(x, dc, db, dw, n, workspace=work)
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        y = S.linear_w4a8(x, dc, db, dw, n, workspace=work)
    for seed in range(3):
        xb, _ = llm_acts(np.random.default_rng(seed), m, k)
        xn = dev(xb)
        x.copy_(xn)
        g.replay()
        want = S.linear_w4a8(xn, dc, db, dw, n)          # eager, own workspace
        torch.cuda.synchronize()
        assert torch.equal(y, want), seed


@pytest.mark.parametrize("m,n,k,fmt_i", [(4000, 4096, 256, 0), (4096, 4100, 128, 0), (4096, 4096, 128, 2), (4090, 4096, 384, 1),
                                          (4096, 4096, 128, 5), (760, 16384, 128, 0)])   # the last: 192 tiles, one round
def test_widest_tile_configuration(S, m, n, k, fmt_i):
    """Problems with at least 256 tiles of 256 x 256 run the widest configuration (wave tiles of 128 x 64, K steps of
    64): ragged last row and column tiles, the published and a generic format, INT32 and all scaling epilogues,
    bit-exact against the oracle."""
    fmt = FORMATS[fmt_i]
    S.set_format(product_format(fmt))
    rng = np.random.default_rng(m + n + k)
    codes, bc, ws, q = random_packed(rng, n, k, fmt)
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    xs = (rng.random(m) * 0.02).astype(F32)
    acc = linear.int_gemm(xq, q)
    wq = S.unpack_i8(dev(codes), dev(bc), n, k)
    assert np.array_equal(host(S.mm_i8_i32(dev(xq), wq)), acc)
    assert np.array_equal(host(S.mm_epi(dev(xq), wq, dev(xs), dev(ws), 1)), linear.epilogue(acc, xs, ws, 1))
    res = bf16.to_bits(rng.standard_normal((m, n)).astype(F32))
    assert np.array_equal(host(S.mm_epi(dev(xq), wq, dev(xs), dev(ws), 2, res=dev(res))),
                          linear.epilogue(acc, xs, ws, 2, res))
    if n % 8 == 0:
        with np.errstate(all="ignore"):
            assert np.array_equal(host(S.mm_epi(dev(xq), wq, dev(xs), dev(ws), 3)), linear.epilogue(acc, xs, ws, 3))
    S.set_format(product_format(layout.DEFAULT))


@pytest.mark.parametrize("name,n,k", [("qkv", 4096, 2048), ("o_proj", 2048, 2048), ("gate_up", 12288, 2048), ("down", 2048, 6144)])
def test_config1_m8192_and_m512_equal_row_blocks_of_m2048(S, name, n, k):
    """BASELINE config 1's other token counts.  A row of the output depends on its own activation row only, so the
    M = 8192 launch (widest tiles) and the M = 512 launches (narrow tiles) must reproduce, bit for bit, the rows that
    M = 2048 launches (checked against the oracle above) give for the same activations."""
    rng = np.random.default_rng(n + k)
    codes, bc, ws, _ = random_packed(rng, n, k)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    x = torch.randn((8192, k), device="cuda", generator=torch.Generator(device="cuda").manual_seed(n)).to(torch.bfloat16)
    big = S.linear_w4a8(x, dc, db, dw, n)
    for r0 in range(0, 8192, 2048):
        assert torch.equal(big[r0:r0 + 2048], S.linear_w4a8(x[r0:r0 + 2048].contiguous(), dc, db, dw, n)), (name, r0)
    for r0 in (0, 3584):
        assert torch.equal(big[r0:r0 + 512], S.linear_w4a8(x[r0:r0 + 512].contiguous(), dc, db, dw, n)), (name, r0)


@pytest.mark.parametrize("name,m,n,k", [("o_proj", 512, 2048, 2048), ("o_proj", 8192, 2048, 2048), ("down", 512, 2048, 6144),
                                        ("qkv", 512, 4096, 2048)])
def test_config1_m512_and_m8192_against_the_oracle(S, name, m, n, k):
    """BASELINE config 1's other token counts held against the oracle directly (not through another launch): the
    one-call layer with weights and activations generated as config 0 prescribes, every INT32 accumulator and every
    bf16 output bit for bit, and the 1e-2 relative Frobenius bound of the float path."""
    rng = np.random.default_rng(7 * m + n + k)
    codes, bc, ws, q = layout.quantize(llm_weights(rng, n, k))
    bits, x = llm_acts(rng, m, k)
    xq_ref, xs_ref = linear.act_quant(x)
    acc_ref = linear.int_gemm(xq_ref, q)
    dc, db, dw = dev(codes), dev(bc), dev(ws)
    xq, xs = S.act_quant(dev(bits), Mp=m)
    assert np.array_equal(host(S.mm_i8_i32(xq, S.unpack_i8(dc, db, n, k))), acc_ref)
    y = host(S.linear_w4a8(dev(bits), dc, db, dw, n))
    assert np.array_equal(y, linear.epilogue(acc_ref, xs_ref, ws, 1))
    assert linear.rel_fro(bf16.from_bits(y), linear.float_reference(x, q, ws)) < 1e-2   # the north star's tolerance


@pytest.mark.parametrize("m,n,k", [(512, 2048, 6144), (131, 2048, 2048), (192, 4096, 1024), (16, 256, 1024), (200, 1000, 1280),
                                   (64, 16384, 768), (100, 2048, 6144), (3, 8, 512)])
@pytest.mark.parametrize("fmt_i", [0, 1, 2, 5])
def test_few_tiles_two_k_groups(S, m, n, k, fmt_i):
    """Problems with no more 64x64 tiles than CUs run two K groups per tile, with no more 64x32 tiles than CUs (and K a
    multiple of 512) four, whose INT32 partial sums meet in LDS: INT32 output and every epilogue against the oracle,
    from one K step per group to 24, in four formats (one per decode path of the kernel), from INT8 and from packed
    weights."""
    fmt = FORMATS[fmt_i]
    rng = np.random.default_rng(m + n + k + fmt_i)
    codes, bc, _, q = random_packed(rng, n, k, fmt)
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    xq[0] = 127
    xs = (np.abs(rng.standard_normal(m)) * 1e-3).astype(F32)
    ws = (np.abs(rng.standard_normal(n)) * 1e-4).astype(F32)
    res = bf16.to_bits(rng.standard_normal((m, n)).astype(F32))
    acc = linear.int_gemm(xq, q)
    S.set_format(product_format(fmt))
    try:
        for lazy in (False, True):
            wq = S.unpack_i8(dev(codes), dev(bc), n, k, lazy=lazy)
            assert np.array_equal(host(S.mm_i8_i32(dev(xq), wq)), acc)
            assert np.array_equal(host(S.mm_epi(dev(xq), wq, dev(xs), dev(ws), 1)), linear.epilogue(acc, xs, ws, 1))
            assert np.array_equal(host(S.mm_epi(dev(xq), wq, dev(xs), dev(ws), 2, res=dev(res))),
                                  linear.epilogue(acc, xs, ws, 2, res))
            assert np.array_equal(host(S.mm_epi(dev(xq), wq, dev(xs), dev(ws), 3)), linear.epilogue(acc, xs, ws, 3))
    finally:
        S.set_format(product_format(layout.DEFAULT))


@pytest.mark.parametrize("m,k", [(200, 2048), (2048, 6144), (1, 1024), (70, 160), (33, 3072), (130, 8192), (64, 96)])
def test_act_quant_blocked(S, m, k):
    """The blocked quantizer writes the codes of act_quant, block by block, and the same scales."""
    rng = np.random.default_rng(m + k)
    bits, x = llm_acts(rng, m, k)
    if m > 3:
        bits[3] = 0
        x[3] = 0
    mp = (m + 31) // 32 * 32
    bx, xs = S.act_quant_blocked(dev(bits), mp)
    rq, rs = linear.act_quant(x, mp)
    assert np.array_equal(host(bx.data), blocked_layout(rq)) and np.array_equal(host(xs), rs)
    assert np.array_equal(host(bx.rows()), rq)


@pytest.mark.parametrize("m,n,k,fmt_i", [(2048, 4096, 2048, 0), (2048, 2048, 6144, 0), (4096, 8192, 512, 1), (300, 1000, 1280, 0),
                                         (70, 512, 256, 5), (1, 8, 128, 0), (2049, 4100, 384, 2), (515, 3072, 1024, 1),
                                         (8192, 2048, 256, 0), (515, 1000, 4096, 1), (130, 2048, 8192, 3), (1024, 4096, 2048, 0),
                                         (100, 128, 512, 0), (128, 32768, 256, 0)])
def test_blocked_activations_give_the_same_gemm(S, m, n, k, fmt_i):
    """Activations in the blocked layout (fragments loaded from memory by the large tiles: 256x256, 256x128, 128x128 or
    256x64 by shape) against the same activations by rows: INT32 and every epilogue bit for bit, ragged M and N included; the
    INT32 result of the smaller shapes also against the oracle directly."""
    fmt = FORMATS[fmt_i]
    rng = np.random.default_rng(m + n + k)
    codes, bc, ws, q = random_packed(rng, n, k, fmt)
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    xq[0] = 127
    mp = (m + 31) // 32 * 32
    padded = np.zeros((mp, k), np.int8)
    padded[:m] = xq
    xs = (np.abs(rng.standard_normal(m)) * 1e-3 + 1e-5).astype(F32)
    res = dev(bf16.to_bits(rng.standard_normal((m, n)).astype(F32)))
    S.set_format(product_format(fmt))
    try:
        wq = S.unpack_i8(dev(codes), dev(bc), n, k, lazy=True)
        rows, blocks = dev(xq), S.BlockedXq(dev(blocked_layout(padded)), m, k)
        acc = S.mm_i8_i32(blocks, wq)
        assert torch.equal(acc, S.mm_i8_i32(rows, wq))
        if m * n * k <= 300 * 1000 * 1280:
            assert np.array_equal(host(acc), linear.int_gemm(xq, q))
        for epi in (1, 2, 3):
            if epi == 3 and n % 8:
                continue
            a = S.mm_epi(blocks, wq, dev(xs), dev(ws), epi, res=res if epi == 2 else None)
            b = S.mm_epi(rows, wq, dev(xs), dev(ws), epi, res=res if epi == 2 else None)
            assert torch.equal(a, b), epi
    finally:
        S.set_format(product_format(layout.DEFAULT))


def test_blocked_activations_need_packed_weights(S):
    bx, _ = S.act_quant_blocked(torch.zeros((32, 128), dtype=torch.bfloat16, device="cuda"), 32)
    with pytest.raises(ValueError):
        S.mm_i8_i32(bx, torch.zeros((8, 128), dtype=torch.int8, device="cuda"))


def test_random_shapes_formats_and_epilogues(S):
    """Fifty seeded random problems (ragged M and N, K of 1 to 8 K steps, every test format, every epilogue) through
    the dense GEMM (activations by rows and in blocks), and row 0 of each through the GEMV: bit-exact against the oracle."""
    from mxfp4_int8_m5_amd import sc_decode as G
    rng = np.random.default_rng(2024)
    done = 0
    try:
        while done < 50:
            fmt = FORMATS[int(rng.integers(0, len(FORMATS)))]
            m, n, k = int(rng.integers(1, 700)), int(rng.integers(1, 180)) * 4, int(rng.integers(1, 9)) * 128
            if (k // fmt.block * fmt.bc_bits) % 8:
                continue
            pf = product_format(fmt)
            S.set_format(pf)
            codes, bc, ws, q = random_packed(rng, n, k, fmt)
            xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
            xs = (np.abs(rng.standard_normal(m)) * 1e-2 + 1e-4).astype(F32)
            epi = int(rng.integers(0, 4))
            if epi == 3 and n % 8:
                epi = 1
            acc = linear.int_gemm(xq, q)
            res = bf16.to_bits(rng.standard_normal((m, n)).astype(F32))
            wq = S.unpack_i8(dev(codes), dev(bc), n, k)
            if epi == 0:
                got, want = host(S.mm_i8_i32(dev(xq), wq)), acc
            else:
                got = host(S.mm_epi(dev(xq), wq, dev(xs), dev(ws), epi, res=dev(res) if epi == 2 else None))
                want = linear.epilogue(acc, xs, ws, epi, res if epi == 2 else None)
            assert np.array_equal(got[:m], want), (done, fmt, m, n, k, epi)
            mp = (m + 31) // 32 * 32                      # the same problem from blocked activations
            padded = np.zeros((mp, k), np.int8)
            padded[:m] = xq
            blocks = S.BlockedXq(dev(blocked_layout(padded)), m, k)
            if epi == 0:
                got_b = host(S.mm_i8_i32(blocks, wq))
            else:
                got_b = host(S.mm_epi(blocks, wq, dev(xs), dev(ws), epi, res=dev(res) if epi == 2 else None))
            assert np.array_equal(got_b[:m], want), ("blocked", done, fmt, m, n, k, epi)
            ev = epi if epi else 1
            y = host(G.gemv(dev(xq[0]), dev(codes), dev(bc), dev(xs[:1]), dev(ws), n, ev, res=dev(res[0]) if ev == 2 else None,
                            fmt=pf))
            wantv = linear.gemv(xq[0], xs[0], q, ws, ev, res[0] if ev == 2 else None)
            assert np.array_equal(y.reshape(-1), np.asarray(wantv).reshape(-1)), (done, fmt, n, k, ev)
            done += 1
    finally:
        S.set_format(product_format(layout.DEFAULT))
