"""Writes tests/golden/quantizer_vectors.npz: inputs and outputs of the reference's own
quantizers, which only the reference itself can pin bit for bit (float32 division followed by
numpy's round-half-even at exact .5 ties):

    repack_experts.quantize_affine_pack   (finchmoe/repack_experts.py:302-333)   bits 3, 4
    repack_experts.quantize_affine_3bit   (finchmoe/repack_experts.py:260-276)   bits 3
    quantize_model.quantize_affine        (finchmoe/quantize_model.py:19-47)     bits 4, 8
    quantize_non_experts.quantize_affine  (finchmoe/quantize_non_experts.py:40-69) bits 4, 8

Runs only in the build container, where /root/reference exists (the three modules define
functions and constants at import, nothing else); the fixture it writes is data and is what
the tests read.  Usage: python tests/golden/make_quantizer_vectors.py
"""
import os
import sys

import numpy as np

REF = "/root/reference/finchmoe"
HERE = os.path.dirname(os.path.abspath(__file__))


def inputs():
    rng = np.random.default_rng(20240607)
    rows = []
    rows.append((rng.standard_normal((6, 256)) * 0.02).astype(np.float32))          # weight-like
    rows.append((rng.standard_normal((2, 256)) * 3.0 + 1.5).astype(np.float32))     # wide, offset
    t = np.zeros((4, 256), np.float32)
    # exact .5 ties: min 0, max = 2^bits - 1 for bits 3 / 4 / 8 puts every k + 0.5 on a tie
    for g, top in enumerate((7.0, 15.0, 255.0, 7.0)):
        grp = np.arange(64, dtype=np.float32) % (top + 1)
        grp = np.where(np.arange(64) % 2 == 1, np.minimum(grp + 0.5, top), grp).astype(np.float32)
        grp[0], grp[63] = 0.0, top
        t[0, 64 * g:64 * g + 64] = grp
        t[1, 64 * g:64 * g + 64] = -grp                       # negative range, bias = -top
        t[2, 64 * g:64 * g + 64] = grp * np.float32(0.125)    # ties survive a power-of-two scale
    t[3, 0:64] = 0.37                                         # constant group: scale clamps to 1e-8
    t[3, 64:128] = np.linspace(1.0, 1.0 + 3e-8, 64, dtype=np.float32)   # range under the clamp
    t[3, 128:192] = rng.standard_normal(64).astype(np.float32) * 1e-3
    t[3, 128] = 40.0                                          # one outlier stretches the group
    t[3, 192:256] = -np.abs(rng.standard_normal(64)).astype(np.float32) * 1e4
    rows.append(t)
    return np.ascontiguousarray(np.concatenate(rows, 0))


def main():
    sys.path.insert(0, REF)
    import repack_experts
    import quantize_model
    import quantize_non_experts
    w = inputs()
    out = {"w": w}
    for bits in (3, 4):
        p, s, b = repack_experts.quantize_affine_pack(w.copy(), bits)
        out["pack%d_w" % bits] = np.ascontiguousarray(p).view(np.uint8).reshape(w.shape[0], -1)
        out["pack%d_s" % bits], out["pack%d_b" % bits] = s, b
    p, s, b = repack_experts.quantize_affine_3bit(w.copy())
    out["q3_w"], out["q3_s"], out["q3_b"] = np.ascontiguousarray(p), s, b
    for name, mod in (("qm", quantize_model), ("qne", quantize_non_experts)):
        for bits in (4, 8):
            p, s, b = mod.quantize_affine(w.copy(), bits)
            out["%s%d_w" % (name, bits)] = np.ascontiguousarray(p).view(np.uint8).reshape(w.shape[0], -1)
            out["%s%d_s" % (name, bits)], out["%s%d_b" % (name, bits)] = s, b
    path = os.path.join(HERE, "quantizer_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes;", len(out), "arrays")


if __name__ == "__main__":
    main()
