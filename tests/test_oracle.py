"""Pins the CPU oracle (oracle/np_oracle.c) independently of itself.

Checks, per oracle function:
* golden vectors made by big-integer packing / numpy arithmetic (tests/golden);
* the known answers the reference's own tests state
  ([3, 11] at 4 bits -> 0xB3; byte count ceil(n*b/8); code 15, zp 2, scale 1 -> 13;
  an underflowed scale decodes to 0; the bits_for table);
* closed forms and invariants (pack . unpack = id, codebook permutation invariance,
  zero residual == plain decode, linearity of the contraction);
* the torch restatement of the reference CPU path (oracle/torch_path.py), a second
  independently written implementation.
"""

import math
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from oracle import torch_path

G = np.load(Path(__file__).parent / "golden" / "vectors.npz")
VQ_NAMES = sorted({k.split("/")[0] for k in G.files if k.startswith("vq_")})
Q_NAMES = sorted({k.split("/")[0] for k in G.files if k[0] == "q" and "/" in k})
CODES = {"f16": orc.DT_F16, "bf16": orc.DT_BF16, "f32": orc.DT_F32}


# ------------------------------------------------------------------ streams ---


@pytest.mark.parametrize("bits", range(4, 21))
def test_unpack_and_pack_match_bigint_streams(oracle_lib, bits):
    idx, packed = G[f"stream_b{bits}/idx"], G[f"stream_b{bits}/packed"]
    assert packed.size == math.ceil(idx.size * bits / 8)
    assert np.array_equal(oracle_lib.unpack_indices(packed, bits, idx.size), idx)
    assert np.array_equal(oracle_lib.pack_indices(idx, bits), packed)


def test_reference_known_answers_for_packing(oracle_lib):
    # tests/transforms/test_vq_packing.py:100-105 of the reference
    assert oracle_lib.pack_indices(np.array([3, 11]), 4).tolist() == [0xB3] == G["kat/pack_3_11_b4"].tolist()
    # tests/transforms/test_vq_packing_extended.py:80-89: exactly ceil(n*bits/8) bytes
    for bits in range(4, 17):
        assert oracle_lib.pack_indices(np.zeros(100, dtype=np.int64), bits).size == math.ceil(100 * bits / 8)
    # :92-99 maximum index survives
    for bits in range(4, 17):
        mx = (1 << bits) - 1
        p = oracle_lib.pack_indices(np.array([mx, 0, mx, 0]), bits)
        assert oracle_lib.unpack_indices(p, bits, 4).tolist() == [mx, 0, mx, 0]


def test_bits_for_table(oracle_lib):
    # tests/transforms/test_vq_packing_extended.py:21-60 of the reference
    table = {2: 4, 16: 4, 17: 5, 32: 5, 33: 6, 64: 6, 65: 7, 128: 7, 129: 8, 256: 8, 257: 9, 512: 9,
             513: 10, 1024: 10, 1025: 11, 2048: 11, 4096: 12, 8192: 13, 16384: 14, 32768: 15, 65536: 16}
    for nc, b in table.items():
        assert oracle_lib.bits_for(nc) == b
    for nc in [3, 5, 10, 20, 100, 300, 1000, 5000, 50000]:
        assert oracle_lib.bits_for(nc) == max(4, math.ceil(math.log2(nc)))
    for bad in (0, 1, (1 << 20) + 1):
        with pytest.raises(ValueError):
            oracle_lib.bits_for(bad)


def test_unpack_rejects_short_stream(oracle_lib):
    with pytest.raises(ValueError):
        oracle_lib.unpack_indices(np.zeros(3, dtype=np.uint8), 12, 3)


@pytest.mark.parametrize("bits", [5, 6, 7, 9, 10, 12, 14])
def test_odd_counts_round_trip(oracle_lib, bits):
    rng = np.random.default_rng(bits)
    for n in [1, 3, 7, 13, 33, 99]:
        idx = rng.integers(0, 1 << bits, size=n)
        assert np.array_equal(oracle_lib.unpack_indices(oracle_lib.pack_indices(idx, bits), bits, n), idx)


# ------------------------------------------------------------------- decode ---


@pytest.mark.parametrize("name", VQ_NAMES)
@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_vq_decode_matches_golden(oracle_lib, name, dt):
    n, k, vl, bits, nc = G[f"{name}/meta"]
    w = oracle_lib.vq_decode(G[f"{name}/packed"], int(bits), G[f"{name}/cb"], int(n), int(k), CODES[dt])
    ref = G[f"{name}/w_{dt}"]
    assert w.dtype == ref.dtype and np.array_equal(w, ref)


def test_vq_decode_matches_torch_cast_rules(oracle_lib):
    """bf16 = RNE of the exact value, incl. ties, subnormals, inf: torch's .to() is the referee."""
    bits_pat = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    keep = ((bits_pat & 0x7C00) != 0x7C00) | ((bits_pat & 0x3FF) == 0)  # drop NaNs
    cb_bits = bits_pat[keep]
    cb_bits = cb_bits[: (cb_bits.size // 8) * 8].reshape(-1, 8)
    nc = cb_bits.shape[0]
    idx = np.arange(nc)
    packed = oracle_lib.pack_indices(idx, 13)
    cb_t = orc.from_bits(cb_bits, torch.float16)
    for dt in (torch.bfloat16, torch.float32, torch.float16):
        w = oracle_lib.vq_decode(packed, 13, cb_bits, nc, 8, orc.torch_dtype_code(dt))
        assert np.array_equal(w, orc.to_bits(cb_t.to(dt)))


def test_vq_decode_codebook_permutation_invariance(oracle_lib):
    rng = np.random.default_rng(5)
    cb = (rng.standard_normal((64, 8))).astype(np.float16)
    idx = rng.integers(0, 64, size=40)
    perm = rng.permutation(64)
    inv = np.argsort(perm)
    a = oracle_lib.vq_decode(oracle_lib.pack_indices(idx, 6), 6, cb.view(np.uint16), 5, 64, orc.DT_F16)
    b = oracle_lib.vq_decode(oracle_lib.pack_indices(inv[idx], 6), 6, cb[perm].view(np.uint16), 5, 64, orc.DT_F16)
    assert np.array_equal(a, b)


def test_vq_decode_out_of_range_index(oracle_lib):
    with pytest.raises(IndexError):
        oracle_lib.vq_decode(np.array([0xFF], dtype=np.uint8), 8, np.zeros((4, 8), np.uint16), 1, 8, orc.DT_F16)


@pytest.mark.parametrize("name", Q_NAMES)
@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_q_decode_matches_golden(oracle_lib, name, dt):
    n, k, nbits, gs, asym = G[f"{name}/meta"]
    zp = G[f"{name}/zp"] if asym else None
    w = oracle_lib.q_decode(G[f"{name}/blob"], G[f"{name}/scale"], zp, int(nbits), int(gs), CODES[dt])
    assert np.array_equal(w, G[f"{name}/w_{dt}"])


def test_q_decode_reference_known_answers(oracle_lib):
    # tests/test_quantized_weight_regressions.py:848-859 of the reference
    blob = np.full((2, 16), 0xFF, dtype=np.uint8)  # 32 codes of 15 per row
    scale = np.array([1e-12, 1.0], dtype=np.float16).view(np.uint16)
    zp = np.array([2.0, 2.0], dtype=np.float16).view(np.uint16)
    w = oracle_lib.q_decode(blob, scale, zp, 4, 32, orc.DT_F32)
    assert (w[0] == 0).all() and (w[1] == 13).all()
    # nibble order: byte = lo | hi << 4 (neuropress/t2n/packing.py:10-14)
    w = oracle_lib.q_decode(np.array([[0x2F] * 16], dtype=np.uint8), np.array([1.0], np.float16).view(np.uint16),
                            None, 4, 32, orc.DT_F32)
    assert w[0, 0] == 15 - 8 and w[0, 1] == 2 - 8


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_rvq_decode_matches_golden_and_reduces_to_vq(oracle_lib, dt):
    n, k, vl, bm, br = (int(v) for v in G["rvq/meta"])
    w = oracle_lib.rvq_decode(G["rvq/pm"], bm, G["rvq/pr"], br, G["rvq/cbm"], G["rvq/cbr"],
                              G["rvq/scale"], G["rvq/wbias"], n, k, CODES[dt])
    assert np.array_equal(w, G[f"rvq/w_{dt}"])
    # zero residual codebook, no scale / bias  ==  single-codebook decode
    # (compared as f32 values: -0 + 0 = +0 is the one bit pattern that may change)
    zero_cb = np.zeros_like(G["rvq/cbr"])
    a = oracle_lib.rvq_decode(G["rvq/pm"], bm, G["rvq/pr"], br, G["rvq/cbm"], zero_cb, None, None, n, k, orc.DT_F32)
    b = oracle_lib.vq_decode(G["rvq/pm"], bm, G["rvq/cbm"], n, k, orc.DT_F32)
    assert np.array_equal(a, b)
    one = np.full(n, 0x3C00, dtype=np.uint16)
    c = oracle_lib.rvq_decode(G["rvq/pm"], bm, G["rvq/pr"], br, G["rvq/cbm"], G["rvq/cbr"], one, None, n, k, CODES[dt])
    d = oracle_lib.rvq_decode(G["rvq/pm"], bm, G["rvq/pr"], br, G["rvq/cbm"], G["rvq/cbr"], None, None, n, k, CODES[dt])
    assert np.array_equal(c, d)  # scale 1.0 is the identity


# -------------------------------------------------------------- contraction ---


@pytest.mark.parametrize("name", VQ_NAMES)
def test_linear_matches_numpy_float64(oracle_lib, name):
    y = oracle_lib.linear_f64(G[f"{name}/x"], orc.DT_F16, G[f"{name}/w_f16"], orc.DT_F16, G[f"{name}/bias"], orc.DT_F16)
    assert np.allclose(y, G[f"{name}/y_f16w"], rtol=1e-12, atol=1e-12)


def test_linear_is_linear_and_transposition_sensitive(oracle_lib):
    rng = np.random.default_rng(11)
    x1 = rng.standard_normal((2, 24)).astype(np.float32)
    x2 = rng.standard_normal((2, 24)).astype(np.float32)
    w = rng.standard_normal((5, 24)).astype(np.float32)
    f = lambda x: oracle_lib.linear_f64(x, orc.DT_F32, w, orc.DT_F32)
    assert np.allclose(f(x1 + x2), f(x1) + f(x2), atol=1e-5)
    assert np.allclose(f(x1), x1.astype(np.float64) @ w.astype(np.float64).T, atol=1e-12)


# ------------------------------------------- the torch restatement agrees too ---


@pytest.mark.parametrize("name", VQ_NAMES)
def test_torch_path_agrees_with_oracle(oracle_lib, name):
    n, k, vl, bits, nc = (int(v) for v in G[f"{name}/meta"])
    packed = torch.from_numpy(G[f"{name}/packed"].copy())
    cb = orc.from_bits(G[f"{name}/cb"], torch.float16)
    x = orc.from_bits(G[f"{name}/x"], torch.float16).float()
    for fast in (False, True):
        y = torch_path.vq_linear_cpu(x, packed, cb, bits, n, k, None, fast_unpack=fast)
        ref = oracle_lib.linear_f64(x.numpy(), orc.DT_F32, G[f"{name}/w_f32"], orc.DT_F32)
        assert np.allclose(y.double().numpy(), ref, atol=1e-4)


@pytest.mark.parametrize("name", Q_NAMES)
def test_torch_q_path_agrees_with_oracle(oracle_lib, name):
    n, k, nbits, gs, asym = (int(v) for v in G[f"{name}/meta"])
    blob = torch.from_numpy(G[f"{name}/blob"].copy())
    scale = orc.from_bits(G[f"{name}/scale"], torch.float16)
    zp = orc.from_bits(G[f"{name}/zp"], torch.float16) if asym else None
    x = orc.from_bits(G[f"{name}/x"], torch.float16).float()
    y = torch_path.q_linear_cpu(x, blob, scale, nbits, gs, zp)
    ref = oracle_lib.linear_f64(x.numpy(), orc.DT_F32, G[f"{name}/w_f32"], orc.DT_F32)
    assert np.allclose(y.double().numpy(), ref, atol=1e-4)
