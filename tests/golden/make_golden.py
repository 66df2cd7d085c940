"""Writes tests/golden/*.npz: input/output vectors of the reference's pure-numpy quantizer and packing modules.

Run ONLY in a container that has the reference checked out (default /root/reference); the reference itself is never
copied or shipped — only the arrays it returns for the inputs generated here.  The functions covered are the ones no
closed form pins: the exponent search with its tie-breaks, the spread constraint, the INT8 embedding, the packed
layouts, and the format-family quantizer's base search.

    python tests/golden/make_golden.py [/path/to/reference]
"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def weight_cases():
    """name -> float64 weight matrix (small; stored in full)."""
    out = {}
    rng = np.random.default_rng(0)
    out["lognormal_cols"] = (rng.standard_normal((64, 1024)) * rng.lognormal(0, 1.0, (1, 1024)))[:16, :512].copy()
    rng = np.random.default_rng(1)
    w = rng.standard_normal((48, 256)) * 0.02
    w[:, rng.choice(256, 2, replace=False)] *= 8
    out["llm_outlier_cols"] = w
    rng = np.random.default_rng(2)
    w = rng.standard_normal((24, 128)) * np.exp2(rng.integers(-12, 12, (24, 4)).repeat(32, 1).astype(np.float64))
    w[3] = 0.0                       # all-zero row
    w[5, 32:64] = 0.0                # all-zero block
    w[7, :] = 0.0
    w[7, 5] = 1e-30                  # single tiny value
    out["wide_exponents_zeros"] = w
    # exact E2M1 midpoints at several scales: ties must go to the lower level
    mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 7.0, 0.0, -0.25, -5.0, -2.5, 4.0, 3.0, 1.0])
    w = np.stack([np.tile(mids, 8) * s for s in (1.0, 0.5, 2.0 ** -7, 3.0, 1.0 / 3.0, 1e-3, 17.0, 2.0 ** 10)])
    out["midpoints"] = w
    return out


def main(ref):
    sys.path.insert(0, os.path.join(ref, "sim"))
    sys.path.insert(0, os.path.join(ref, "e2e"))
    import mx_int8
    import make_testcase
    import sc_format
    import formats
    import pack_format
    import gptq_pack

    g = {}
    # ---- elementwise E2M1 rounding on a dense grid incl. every midpoint and its neighbours
    pts = np.concatenate([np.linspace(-7, 7, 2801), mx_int8._MIDS, np.nextafter(mx_int8._MIDS, 10),
                          np.nextafter(mx_int8._MIDS, -10), -mx_int8._MIDS, [0.0, -0.0, 1e-300, 6.0, 1e9, -1e9]])
    g["e2m1_in"], g["e2m1_out"] = pts, mx_int8.round_e2m1(pts)

    # ---- quantizer on small matrices, stored in full
    for name, w in weight_cases().items():
        g[f"w/{name}"] = w
        for rule in ("spec", "search"):
            e = mx_int8.block_exponents(w, rule)
            g[f"e_{rule}/{name}"] = e
        ec = mx_int8.constrain_spread(w, mx_int8.block_exponents(w, "search"))
        g[f"e_sc/{name}"] = ec
        wdq, v = mx_int8.dequant_mx(w, ec)
        g[f"v/{name}"], g[f"wdq/{name}"] = v, wdq
        q, sc = mx_int8.embed_int8(v, ec)
        g[f"q/{name}"], g[f"sc/{name}"] = q, sc
        packed, shifts, wscale, qw = make_testcase.pack(w)
        g[f"packed/{name}"], g[f"shifts/{name}"], g[f"wscale/{name}"], g[f"qw/{name}"] = packed, shifts, wscale, qw
        p2 = gptq_pack.pack_ve(v, ec)
        assert all(np.array_equal(a, b) for a, b in zip(p2, (packed, shifts, wscale, qw)))
        codes, bc, ws, _ = sc_format.quantize(w)
        g[f"codes/{name}"], g[f"bcodes/{name}"] = codes, bc
        assert np.array_equal(sc_format.decode_numpy(codes, bc, *w.shape), qw)

    # ---- larger seeded matrices: only digests are stored; the test regenerates the input from the seed
    big = {}
    rng = np.random.default_rng(0)
    big["selftest_mx_int8"] = rng.standard_normal((64, 1024)) * rng.lognormal(0, 1.0, (1, 1024))
    rng = np.random.default_rng(0)
    big["selftest_sc_format"] = rng.standard_normal((64, 512)) * 0.02 * rng.lognormal(0, 0.3, (1, 512))
    rng = np.random.default_rng(0)
    big["test_sc_kernels_384x2048"] = rng.standard_normal((384, 2048)) * 0.02 * rng.lognormal(0, 0.3, (1, 2048))
    rng = np.random.default_rng(7)
    w = rng.standard_normal((256, 2048)) * 0.02
    w[:, rng.choice(2048, 10, replace=False)] *= 8
    big["config0_like_256x2048"] = w
    for name, w in big.items():
        packed, shifts, wscale, qw = make_testcase.pack(w)
        g[f"sha/{name}"] = np.array([sha(packed), sha(shifts), sha(wscale), sha(qw)])

    # ---- packed layout on random codes, the five formats of the reference's format test
    fmts = [dict(), dict(block=16), dict(block=32, mult=(1, 2, 3, 4)),
            dict(block=16, mult=(1, 2, 3, 4, 5, 6, 8, 10), bc_bits=4),
            dict(block=32, code_mag=(0, 1, 2, 3, 4, 5, 6, 7), mult=(1, 3, 9, 15))]
    rng = np.random.default_rng(3)
    for i, kw in enumerate(fmts):
        f = sc_format.Format(**kw)
        n, k = 8, 256
        c4 = rng.integers(0, 16, (n, k)).astype(np.uint8)
        b = rng.integers(0, len(f.mult), (n, k // f.block)).astype(np.uint8)
        codes, bc, ws = sc_format.pack_rows(c4, b, np.abs(rng.standard_normal(n)) * 1e-3, f)
        g[f"fmt{i}/c4"], g[f"fmt{i}/b"] = c4, b
        g[f"fmt{i}/codes"], g[f"fmt{i}/bc"], g[f"fmt{i}/ws"] = codes, bc, ws
        g[f"fmt{i}/q"] = sc_format.decode_numpy(codes, bc, n, k, f)

    # ---- format-family quantizer (float32 decisions, row-base search)
    rng = np.random.default_rng(4)
    wf = (rng.standard_normal((24, 256)) * rng.lognormal(0, 1, (1, 256))).astype(np.float32)
    wf[2] = 0
    g["fam/w"] = wf
    for name in ("e2m1/B16/pow2", "e2m1/B16/M1..10", "e2m1/B32/M1..8", "int4/B16/M1..16"):
        fam = formats.FORMATS[name]
        wq, qi, base, scales = formats.quantize(wf, fam)
        key = name.replace("/", "_")
        g[f"fam/{key}/wq"], g[f"fam/{key}/qi"], g[f"fam/{key}/base"], g[f"fam/{key}/scales"] = wq, qi, base, scales
        sf = pack_format.sc_format_of(name)
        codes, bc, ws, stats = pack_format.pack_parts(wq, qi, base, scales, sf)
        assert stats["exact_q"]
        g[f"fam/{key}/codes"], g[f"fam/{key}/bc"], g[f"fam/{key}/ws"] = codes, bc, ws
        g[f"fam/{key}/fmt"] = np.array([sf.block, sf.bc_bits, len(sf.mult)] + list(sf.code_mag) + list(sf.mult))

    # ---- the linear-layer test case make_testcase.main writes (float64 activation quantization, exact GEMM)
    import json
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        make_testcase.main(24, 32, 256, tmp)
        meta = json.load(open(os.path.join(tmp, "meta.json")))
        m, n, k = meta["M"], meta["N"], meta["K"]
        rd = lambda name, dt, shape: np.fromfile(os.path.join(tmp, name + ".bin"), dt).reshape(shape)
        g["layer/x"] = rd("x", np.float16, (m, k))
        g["layer/codes"] = rd("codes", np.uint8, (n, k // 2))
        g["layer/shifts"] = rd("shifts", np.uint8, (n, k // 32))
        g["layer/shifts2"] = rd("shifts2", np.uint8, (n, k // 128))
        g["layer/wscale"] = rd("wscale", np.float32, (n,))
        g["layer/xq"] = rd("xq", np.int8, (m, k))
        g["layer/xscale"] = rd("xscale", np.float32, (m,))
        g["layer/wq"] = rd("wq", np.int8, (n, k))
        g["layer/y_ref"] = rd("y_ref", np.float32, (m, n))

    np.savez_compressed(os.path.join(HERE, "reference_vectors.npz"), **g)
    print(f"wrote {len(g)} arrays, {os.path.getsize(os.path.join(HERE, 'reference_vectors.npz')) / 1024:.0f} KiB")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
