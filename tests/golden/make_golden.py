"""Writes tests/golden/vectors.npz: small known-answer vectors for the path.

The reference ships no golden files for this path (its tests synthesise every
input), and it cannot be imported here (Python >= 3.13 syntax and an absent
third-party dependency), so these vectors are produced by implementations that
share no code with ``oracle/np_oracle.c`` or with the HIP kernels:

* index streams: Python big-integer arithmetic,
  ``stream = sum(idx[i] << (i*bits))`` written little-endian -- the closed form
  stated at neuropress/transforms/vq_packing.py:70-78;
* decoded weights: numpy fancy indexing on float16 arrays and numpy's own
  float16 -> float32 cast; bfloat16 by explicit round-to-nearest-even integer
  arithmetic on the float32 bits;
* int4 decode: numpy float32 arithmetic ``(q - zp) * scale``;
* residual VQ: numpy float16 arithmetic, one op at a time;
* outputs: numpy float64 matmul.

Run from the repo root:  python tests/golden/make_golden.py
"""

from __future__ import annotations

from pathlib import Path

import numpy as np

OUT = Path(__file__).resolve().parent / "vectors.npz"


def pack_bigint(idx, bits):
    acc = 0
    for i, v in enumerate(idx):
        acc |= int(v) << (i * bits)
    n_bytes = (len(idx) * bits + 7) // 8
    return np.frombuffer(acc.to_bytes(n_bytes, "little"), dtype=np.uint8).copy()


def f32_to_bf16_bits(a):
    x = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    x = x + 0x7FFF + ((x >> 16) & 1)
    return (x >> 16).astype(np.uint16)


def cast_from_f16(w16, code):
    if code == 0:
        return w16.view(np.uint16)
    if code == 1:
        return f32_to_bf16_bits(w16.astype(np.float32))
    return w16.astype(np.float32)


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    # --- VQ cases: (name, N, K, VL, bits, NC) ---
    vq_cases = [
        ("vq_b4", 6, 16, 4, 4, 16), ("vq_b8", 5, 16, 8, 8, 256), ("vq_b10", 7, 24, 4, 10, 1000),
        ("vq_b12", 5, 32, 8, 12, 1500), ("vq_b14", 3, 40, 8, 14, 1200), ("vq_b15", 3, 24, 8, 15, 900),
        ("vq_b16", 4, 64, 8, 16, 1100), ("vq_b5", 3, 12, 4, 5, 32), ("vq_b9", 9, 8, 8, 9, 500),
    ]
    for name, n, k, vl, bits, nc in vq_cases:
        cb = (rng.standard_normal((nc, vl)) * 0.5).astype(np.float16)
        idx = rng.integers(0, nc, size=n * k // vl)
        idx[0], idx[-1] = nc - 1, nc - 1  # the largest index at both ends of the stream
        packed = pack_bigint(idx, bits)
        w16 = cb[idx].reshape(n, k)
        x = rng.standard_normal((3, k)).astype(np.float16)
        bias = rng.standard_normal(n).astype(np.float16)
        y = x.astype(np.float64) @ w16.astype(np.float64).T + bias.astype(np.float64)
        out.update({
            f"{name}/meta": np.array([n, k, vl, bits, nc]), f"{name}/cb": cb.view(np.uint16),
            f"{name}/idx": idx.astype(np.int64), f"{name}/packed": packed,
            f"{name}/w_f16": cast_from_f16(w16, 0), f"{name}/w_bf16": cast_from_f16(w16, 1),
            f"{name}/w_f32": cast_from_f16(w16, 2), f"{name}/x": x.view(np.uint16),
            f"{name}/bias": bias.view(np.uint16), f"{name}/y_f16w": y,
        })
    # --- full-range index streams for every width (largest index, odd counts) ---
    for bits in range(4, 21):
        n = 67 if bits != 4 else 68
        idx = rng.integers(0, 1 << bits, size=n)
        idx[:4] = [(1 << bits) - 1, 0, (1 << bits) - 1, 0]
        out[f"stream_b{bits}/idx"] = idx.astype(np.int64)
        out[f"stream_b{bits}/packed"] = pack_bigint(idx, bits)
    # --- known answers the reference's tests state literally ---
    out["kat/pack_3_11_b4"] = pack_bigint([3, 11], 4)  # == [0xB3]
    # --- int4 / n-bit group affine: (name, N, K, nbits, gs, asym) ---
    for name, n, k, nbits, gs, asym in [("q4_sym", 5, 64, 4, 32, False), ("q4_asym", 4, 64, 4, 16, True),
                                        ("q8_sym", 3, 32, 8, 32, False), ("q2_asym", 3, 32, 2, 8, True),
                                        ("q1_sym", 2, 32, 1, 16, False)]:
        vpb = 8 // nbits
        codes = rng.integers(0, 1 << nbits, size=(n, k)).astype(np.uint8)
        blob = np.zeros((n, k // vpb), dtype=np.uint8)
        for i in range(vpb):
            blob |= (codes[:, i::vpb] << (i * nbits)).astype(np.uint8)
        scale = (rng.random(n * k // gs) * 0.019 + 0.001).astype(np.float16)
        zp = (rng.random(n * k // gs) * ((1 << nbits) - 1)).astype(np.float16) if asym else None
        zpf = zp.astype(np.float32) if asym else np.full(scale.shape, float(1 << (nbits - 1)), np.float32)
        w32 = ((codes.astype(np.float32).reshape(n, k // gs, gs) - zpf.reshape(n, -1, 1))
               * scale.astype(np.float32).reshape(n, -1, 1)).reshape(n, k)
        x = rng.standard_normal((2, k)).astype(np.float16)
        out.update({
            f"{name}/meta": np.array([n, k, nbits, gs, int(asym)]), f"{name}/blob": blob,
            f"{name}/codes": codes, f"{name}/scale": scale.view(np.uint16),
            f"{name}/w_f32": w32, f"{name}/w_f16": w32.astype(np.float16).view(np.uint16),
            f"{name}/w_bf16": f32_to_bf16_bits(w32), f"{name}/x": x.view(np.uint16),
            f"{name}/y_f16w": x.astype(np.float64) @ w32.astype(np.float16).astype(np.float64).T,
        })
        if asym:
            out[f"{name}/zp"] = zp.view(np.uint16)
    # --- residual VQ with row scale / bias, fp16 op by op ---
    n, k, vl, ncm, ncr = 6, 32, 8, 1024, 256
    cbm = (rng.standard_normal((ncm, vl)) * 0.3).astype(np.float16)
    cbr = (rng.standard_normal((ncr, vl)) * 0.05).astype(np.float16)
    im = rng.integers(0, ncm, size=n * k // vl)
    ir = rng.integers(0, ncr, size=n * k // vl)
    s = (rng.random(n) + 0.5).astype(np.float16)
    b = (rng.standard_normal(n) * 0.01).astype(np.float16)
    w = (cbm[im] + cbr[ir]).astype(np.float16).reshape(n, k)
    w = (w * s[:, None]).astype(np.float16)
    w = (w + b[:, None]).astype(np.float16)
    out.update({
        "rvq/meta": np.array([n, k, vl, 10, 8]), "rvq/cbm": cbm.view(np.uint16), "rvq/cbr": cbr.view(np.uint16),
        "rvq/pm": pack_bigint(im, 10), "rvq/pr": pack_bigint(ir, 8), "rvq/scale": s.view(np.uint16),
        "rvq/wbias": b.view(np.uint16), "rvq/w_f16": w.view(np.uint16),
        "rvq/w_bf16": f32_to_bf16_bits(w.astype(np.float32)), "rvq/w_f32": w.astype(np.float32),
    })
    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(out)} arrays)")


if __name__ == "__main__":
    main()
