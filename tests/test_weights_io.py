"""Host logic of the packed-weight containers and their safetensors form (no GPU): key names and dtypes as the
reference writes them (e2e/fused_olmoe.py:123-128, e2e/pack_format.py:99-108), the byte-shift cache import
(e2e/fused_qwen3.py:62-72), row concatenation with a permutation (e2e/fused_qwen3.py:35-59) and the E8M0 export
(e2e/fused_qwen38.py:319-334), each against the numpy oracle."""
import json
import struct

import numpy as np
import pytest

from oracle import layout, quantizer
from tests.util import llm_weights


@pytest.fixture(scope="module")
def W():
    from mxfp4_int8_m5_amd import sc_weights
    return sc_weights


def quantized(seed, n, k):
    rng = np.random.default_rng(seed)
    return layout.quantize(llm_weights(rng, n, k))


def test_cache_round_trip_keys_and_dtypes(W, tmp_path):
    flat, want = {}, {}
    for i, (n, k) in enumerate([(32, 256), (16, 512)]):
        c, b, s, _ = quantized(i, n, k)
        key = f"layers.{i}.self_attn.q_proj" if i == 0 else f"layers.0.experts.gate_proj.{i}"
        flat[key + ".codes"], flat[key + ".bcodes"], flat[key + ".wscale"] = c, b, s
        want[key] = (c, b, s)
    path = str(tmp_path / "cache.safetensors")
    W.save_cache(path, flat)
    with open(path, "rb") as f:                      # the file itself: dtypes as mx.save_safetensors writes them
        hdr = json.loads(f.read(struct.unpack("<Q", f.read(8))[0]))
    assert {k: v["dtype"] for k, v in hdr.items() if k != "__metadata__"} == {
        k + s: d for k in want for s, d in ((".codes", "U32"), (".bcodes", "U8"), (".wscale", "F32"))}
    got = W.load_cache(path)
    assert sorted(got) == sorted(want)
    for key in want:
        for a, b in zip(got[key], want[key]):
            assert a.dtype == b.dtype and np.array_equal(a, b)


def test_cache_rejects_unknown_suffix_and_missing_parts(W, tmp_path):
    with pytest.raises(ValueError):
        W.save_cache(str(tmp_path / "x.safetensors"), {"layers.0.q.weights": np.zeros(4, np.float32)})
    W.save_cache(str(tmp_path / "y.safetensors"), {"layers.0.q.codes": np.zeros(4, np.uint32)})
    with pytest.raises(KeyError):
        W.load_cache(str(tmp_path / "y.safetensors"))


def test_byte_shift_cache_import(W, tmp_path):
    from safetensors.numpy import save_file
    flat, want = {}, {}
    for gi, paths in enumerate(W.GROUPS.values()):
        for pi, p in enumerate(paths):
            w = llm_weights(np.random.default_rng(10 * gi + pi), 24, 256)
            packed, shifts, ws, q = quantizer.pack(w)
            key = f"layers.0.{p}"
            flat[key + ".codes"], flat[key + ".shifts"], flat[key + ".wscale"] = packed, shifts, ws
            want[key] = q
    path = str(tmp_path / "shift.safetensors")
    save_file(flat, path)
    out = W.load_packed(path, 1)
    assert sorted(out) == sorted(want)
    for key, (codes, bc, ws) in out.items():
        assert np.array_equal(layout.decode(codes, bc, 24, 256), want[key])


def test_packed_weight_concatenation_and_permutation(W):
    parts, qs = [], []
    for i, n in enumerate((32, 16, 16)):
        c, b, s, q = quantized(20 + i, n, 512)
        parts.append((c, b, s))
        qs.append(q)
    perm = np.random.default_rng(0).permutation(64)
    pw = W.PackedWeight(parts, perm=perm, device="cpu")
    assert pw.splits == [32, 16, 16] and pw.N == 64 and pw.K == 512
    codes = pw.codes.numpy().view(np.uint32)
    assert np.array_equal(layout.decode(codes, pw.bcodes.numpy(), 64, 512), np.concatenate(qs)[perm])
    assert np.array_equal(pw.wscale.numpy(), np.concatenate([p[2] for p in parts])[perm])
    assert pw.nbytes() == 64 * 512 // 2 + 64 * 4 + 64 * 4
    handle = pw.unpack()
    assert handle.shape == (64, 512)                 # lazy handle: no INT8 copy is made
    with pytest.raises(ValueError):
        W.PackedWeight([parts[0], quantized(30, 8, 256)[:3]], device="cpu")


def test_mxfp4_scales_match_the_oracle_view(W):
    c, b, s, _ = quantized(40, 48, 1024)
    pw = W.PackedWeight([(c, b, s)], device="cpu")
    e8 = W.mxfp4_scales(pw)
    nib, want = layout.to_mxfp4(c, b, s, 48, 1024)
    assert e8.dtype == np.uint8 and e8.flags["C_CONTIGUOUS"] and np.array_equal(e8, want)
    c2, b2, s2 = layout.from_mxfp4(nib, e8)          # and back: the same packed matrix
    assert np.array_equal(c2, c) and np.array_equal(b2, b) and np.array_equal(s2, s)
    pw.wscale = pw.wscale * 1.5
    with pytest.raises(ValueError):
        W.mxfp4_scales(pw)


def test_shift_layout_round_trip():
    """to_shift_layout undoes from_shift_layout: one shift byte per 32-block <-> four 2-bit codes per byte."""
    from mxfp4_int8_m5_amd import sc_format as F
    rng = np.random.default_rng(3)
    n, k = 24, 512
    codes = rng.integers(0, 2 ** 32, n * k // 8, dtype=np.uint64).astype(np.uint32)
    shifts = rng.integers(0, 4, (n, k // 32)).astype(np.uint8)
    ws = (2.0 ** rng.integers(-12, -4, n)).astype(np.float32)
    c, bc, w = F.from_shift_layout(codes, shifts, ws)
    assert bc.shape == (n, k // 128)
    c2, sh2, w2 = F.to_shift_layout(c, bc, w)
    assert np.array_equal(c2, codes) and np.array_equal(sh2, shifts) and np.array_equal(w2, ws)
    assert sh2.dtype == np.uint8 and c2.dtype == np.uint32


def test_read_checkpoint_directory(tmp_path):
    import json
    import torch
    from safetensors.torch import save_file
    from mxfp4_int8_m5_amd import fused_qwen3 as Q
    cfg = dict(hidden_size=64, intermediate_size=128, num_hidden_layers=1, num_attention_heads=4, num_key_value_heads=2,
               rms_norm_eps=1e-5, rope_theta=10000.0, vocab_size=50, tie_word_embeddings=False, model_type="qwen3",
               torch_dtype="bfloat16")
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({"model.norm.weight": torch.ones(64), "lm_head.weight": torch.zeros(50, 64)}, str(tmp_path / "a.safetensors"))
    save_file({"model.embed_tokens.weight": torch.zeros(50, 64)}, str(tmp_path / "b.safetensors"))
    args, state = Q.read_checkpoint(str(tmp_path))
    assert args.head_dim == 16 and args.rms_norm_eps == 1e-5 and args.tie_word_embeddings is False
    assert sorted(state) == ["lm_head.weight", "model.embed_tokens.weight", "model.norm.weight"]
    with pytest.raises(FileNotFoundError):
        (tmp_path / "empty").mkdir()
        (tmp_path / "empty" / "config.json").write_text(json.dumps(cfg))
        Q.read_checkpoint(str(tmp_path / "empty"))
