"""The blocked activation layout on the CPU: the test helper that writes it, the product class that reads it back and
the address formula the C header states agree with each other (no GPU)."""
import numpy as np
import torch

from tests.util import blocked_layout


def test_blocked_layout_formula_and_inverse():
    from mxfp4_int8_m5_amd import sc_kernels as S
    rng = np.random.default_rng(0)
    mp, k = 96, 160
    xq = rng.integers(-127, 128, (mp, k)).astype(np.int8)
    flat = blocked_layout(xq)
    assert flat.shape == (mp * k,)
    # include/scmx.h: block (m / 32, k / 32) at ((m / 32) * (K / 32) + k / 32) * 1024, the 16 bytes xq[m, 16 j ...] at
    # ((j % 2) * 32 + m % 32) * 16 inside it
    for m, kk in ((0, 0), (31, 15), (32, 16), (33, 47), (95, 159), (64, 100), (5, 129)):
        j = kk // 16
        at = ((m // 32) * (k // 32) + kk // 32) * 1024 + ((j % 2) * 32 + m % 32) * 16 + kk % 16
        assert flat[at] == xq[m, kk], (m, kk)
    back = S.BlockedXq(torch.from_numpy(flat), mp, k).rows()
    assert np.array_equal(back.numpy(), xq)
