"""Pins of the CPU oracle's number formats, packers and dequant (no GPU).

Each check is chosen so that a plausible mistake (wrong shift, swapped nibble,
dropped bias, wrong group index) fails it; none of them re-types the oracle's
own formula against itself.
"""
import os

import numpy as np
import pytest

from finchmoe_amd import formats as F


def test_bf16_widen_exhaustive(orc):
    """Every bf16 pattern: the fp32 with those top 16 bits (NaN payloads are altered by the
    float return path of ctypes, so NaNs are compared as NaN)."""
    u = np.arange(65536, dtype=np.uint16)
    L = orc.lib()
    got = np.array([L.orc_bf16_to_f32(int(v)) for v in u], np.float32)
    want = (u.astype(np.uint32) << 16).view(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    back = np.array([L.orc_f32_to_bf16_trunc(float(v)) for v in want[~nan][::5]], np.uint16)
    assert np.array_equal(back, u[~nan][::5])


def test_fp16_widen_exhaustive(orc):
    """Every half bit pattern against numpy's IEEE conversion (NaNs compared as NaN)."""
    L = orc.lib()
    u = np.arange(65536, dtype=np.uint16)
    want = u.view(np.float16).astype(np.float32)
    got = np.array([L.orc_fp16_to_f32(int(v)) for v in u], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_fp16_rne_matches_numpy(orc):
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(0.01),
        (rng.standard_normal(20000) * 10.0 ** rng.uniform(-9, 5, 20000)).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25,
                  np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -14, 6.1e-5,
                  1.0009765625, 1.00048828125, 1.00146484375, np.inf, -np.inf], np.float32),
        # exact ties between adjacent halves
        (np.arange(1024, 2048, dtype=np.float32) + 0.5) / np.float32(1024.0),
    ])
    got = orc.f32_to_fp16_rne(vals)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


def test_bf16_rne(orc):
    L = orc.lib()
    rng = np.random.default_rng(2)
    vals = rng.standard_normal(5000).astype(np.float32)
    import torch
    want = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([L.orc_f32_to_bf16_rne(float(v)) for v in vals], np.uint16)
    assert np.array_equal(got, want)


def test_layout_constants(orc):
    """Offsets as literal numbers from the reference (infer.m:174-234,
    repack_experts.py:76-87, 141-151) against the oracle's and the product's arithmetic."""
    ref3 = dict(gate_w=0, gate_s=393216, gate_b=425984, up_w=458752, up_s=851968, up_b=884736,
                down_w=917504, down_s=1310720, down_b=1343488, expert_size=1376256)
    ref4 = dict(gate_w=0, gate_s=524288, gate_b=557056, up_w=589824, up_s=1114112,
                up_b=1146880, down_w=1179648, down_s=1703936, down_b=1736704,
                expert_size=1769472)
    for bits, ref in ((3, ref3), (4, ref4)):
        lo = orc.expert_layout(2048, 512, 64, bits)
        fl = F.expert_layout(2048, 512, bits)
        for k, v in ref.items():
            assert getattr(lo, k) == v, (bits, k)
            assert fl[k] == v, (bits, k)
    # 397B-class shape (repack_experts.py:108-119)
    lo = orc.expert_layout(4096, 1024, 64, 4)
    assert (lo.gate_s, lo.up_w, lo.down_w, lo.down_b, lo.expert_size) == \
        (2097152, 2359296, 4718592, 6946816, 7077888)
    assert 256 * ref3["expert_size"] == 352321536
    assert 40 * 256 * ref3["expert_size"] == 14092861440


def test_pack3_exhaustive(orc):
    """All 2^24 triplets: pack -> bytes are the little-endian 24-bit value; unpack -> the
    codes; and the product's numpy packer agrees."""
    v = np.arange(1 << 24, dtype=np.uint32)
    codes = np.empty((1 << 24, 8), np.uint8)
    for j in range(8):
        codes[:, j] = (v >> (3 * j)) & 7
    packed = orc.pack_3bit(codes)
    want = np.empty((1 << 24, 3), np.uint8)
    want[:, 0] = v & 0xFF
    want[:, 1] = (v >> 8) & 0xFF
    want[:, 2] = (v >> 16) & 0xFF
    assert np.array_equal(packed.reshape(-1, 3), want)
    back = orc.unpack_3bit(packed, codes.size)
    assert np.array_equal(back.reshape(-1, 8), codes)
    sub = codes[::257]
    assert np.array_equal(F.pack_3bit(sub), orc.pack_3bit(sub))


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_pack_u32_fields(orc, bits):
    rng = np.random.default_rng(bits)
    vpu = 32 // bits
    codes = rng.integers(0, 1 << bits, size=(4096, vpu), dtype=np.uint8)
    words = orc.pack_u32(codes, bits)
    # closed form: little-endian positional value
    want = np.zeros(4096, np.uint64)
    for v in range(vpu):
        want += codes[:, v].astype(np.uint64) << np.uint64(v * bits)
    assert np.array_equal(words.astype(np.uint64), want)
    assert np.array_equal(orc.unpack_u32(words, codes.size, bits).reshape(codes.shape), codes)
    assert np.array_equal(F.pack_u32(codes, bits), words)
    # every single field position on its own
    for v in range(vpu):
        one = np.zeros((1, vpu), np.uint8)
        one[0, v] = (1 << bits) - 1
        assert int(orc.pack_u32(one, bits)[0]) == ((1 << bits) - 1) << (v * bits)


@pytest.mark.parametrize("bits", [3, 4, 8])
@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_affine_dequant_exact(orc, bits, dtype):
    """w_f32 == float32(float64(q)*s + b): exactly rounded, compiler independent; the
    codes are the ones that were packed; groups are indexed col // 64."""
    rng = np.random.default_rng(10 * bits + (dtype == "fp16"))
    out_dim, in_dim = 24, 512
    codes, W, S, B = F.synth_affine_tensor(rng, out_dim, in_dim, bits, dtype)
    # edge scales and biases: zero, denormal-ish, large, negative
    if dtype == "bf16":
        S[0, :4] = [0x0000, 0x0001, 0x7F7F, 0x8080]
        B[1, :4] = [0x0000, 0xFF7F, 0x0080, 0x3F80]
        s64 = F.bf16_to_f32(S).astype(np.float64)
        b64 = F.bf16_to_f32(B).astype(np.float64)
    else:
        S[0, :4] = [0x0000, 0x0001, 0x7BFF, 0x8400]
        B[1, :4] = [0x0000, 0xFBFF, 0x0400, 0x3C00]
        s64 = S.view(np.float16).astype(np.float64)
        b64 = B.view(np.float16).astype(np.float64)
    sd = orc.SCALE_BF16 if dtype == "bf16" else orc.SCALE_FP16
    got_codes, got_w = orc.dequant_affine(W, S, B, out_dim, in_dim, bits, scale_dtype=sd)
    assert np.array_equal(got_codes, codes)
    g = np.arange(in_dim) // 64
    with np.errstate(over="ignore", invalid="ignore"):
        want = (codes.astype(np.float64) * s64[:, g] + b64[:, g]).astype(np.float32)
    assert np.array_equal(got_w.view(np.uint32), want.view(np.uint32))


def _np_q4k(blocks):
    """Independent vectorised numpy decode of Q4_K blocks [nb,144] -> float64 [nb,256],
    written from the block description (element e: chunk e//64, half (e//32)&1)."""
    nb = blocks.shape[0]
    d = blocks[:, 0:2].copy().view(np.float16).astype(np.float64)[:, 0]
    dmin = blocks[:, 2:4].copy().view(np.float16).astype(np.float64)[:, 0]
    s = blocks[:, 4:16].astype(np.int64)
    sc = np.empty((nb, 8), np.int64)
    mn = np.empty((nb, 8), np.int64)
    for j in range(8):
        if j < 4:
            sc[:, j] = s[:, j] & 63
            mn[:, j] = s[:, j + 4] & 63
        else:
            sc[:, j] = (s[:, j + 4] & 0xF) | ((s[:, j - 4] >> 6) << 4)
            mn[:, j] = (s[:, j + 4] >> 4) | ((s[:, j] >> 6) << 4)
    qs = blocks[:, 16:144].astype(np.int64)
    y = np.empty((nb, 256), np.float64)
    e = np.arange(256)
    chunk, high, l = e // 64, (e // 32) & 1, e % 32
    nib = (qs[:, 32 * chunk + l] >> (4 * high)) & 0xF
    j = 2 * chunk + high
    y[:] = (d[:, None] * sc[:, j]) * nib - dmin[:, None] * mn[:, j]
    return y


def _np_q6k(blocks):
    nb = blocks.shape[0]
    ql = blocks[:, 0:128].astype(np.int64)
    qh = blocks[:, 128:192].astype(np.int64)
    sc = blocks[:, 192:208].copy().view(np.int8).astype(np.int64)
    d = blocks[:, 208:210].copy().view(np.float16).astype(np.float64)[:, 0]
    e = np.arange(256)
    half, vi = e // 128, e % 128
    nib = (ql[:, 64 * half + (vi & 63)] >> (4 * (vi >> 6))) & 0xF
    hi2 = (qh[:, 32 * half + (vi & 31)] >> (2 * ((vi >> 5) & 3))) & 3
    q = (nib | (hi2 << 4)) - 32
    return d[:, None] * sc[:, 8 * half + (vi >> 4)] * q


@pytest.mark.parametrize("gtype", [12, 14])
def test_gguf_dequant_three_ways(orc, gtype):
    """Row-loop form (infer.m) == word-indexed form (shaders.metal) bit for bit, and both
    equal the float64 evaluation of the block formula (every product is exact in fp32)."""
    rng = np.random.default_rng(gtype)
    rows, in_dim = 8, 512
    W = F.synth_gguf_tensor(rng, rows, in_dim, gtype)
    bsz = 144 if gtype == 12 else 210
    y = orc.gguf_dequant(W, rows, in_dim, gtype)
    blocks = W.reshape(-1, bsz)
    want64 = (_np_q4k(blocks) if gtype == 12 else _np_q6k(blocks)).reshape(rows, in_dim)
    assert np.array_equal(y, want64.astype(np.float32))
    assert np.all(want64.astype(np.float32).astype(np.float64) == want64) or gtype == 12
    for b in range(0, blocks.shape[0], 3):
        for e in range(256):
            v = orc.gguf_block_value_wordform(blocks[b], e, gtype)
            assert np.float32(v).view(np.uint32) == y.reshape(-1, 256)[b, e].view(np.uint32), (b, e)


def test_scale_min_k4_all_fields(orc):
    """Each of the 96 bits of the 12 scale bytes must reach exactly one of the 16 six-bit
    outputs (a wrong shift or mask drops or duplicates one)."""
    L = orc.lib()
    import ctypes as C
    seen = {}
    for bit in range(96):
        s = np.zeros(12, np.uint8)
        s[bit // 8] = 1 << (bit % 8)
        hits = []
        for j in range(8):
            sc, m = C.c_uint8(), C.c_uint8()
            L.orc_get_scale_min_k4(j, s.ctypes.data, C.addressof(sc), C.addressof(m))
            if sc.value:
                hits.append(("sc", j, sc.value))
            if m.value:
                hits.append(("m", j, m.value))
        assert len(hits) == 1, (bit, hits)
        seen[hits[0]] = bit
    assert len(seen) == 96


@pytest.mark.parametrize("bits", [3, 4])
def test_quantizer_roundtrip(orc, bits):
    """Quantizer against a numpy restatement of the same float32 steps and by the bound
    |w - dequant(q)| <= scale/2 (+ bf16 truncation of scale and bias)."""
    rng = np.random.default_rng(bits)
    w = (rng.standard_normal((16, 256)) * 0.02).astype(np.float32)
    codes, S, B = orc.quantize_affine(w, bits)
    maxv = (1 << bits) - 1
    wg = w.reshape(16, 4, 64)
    lo, hi = wg.min(2), wg.max(2)
    scale = np.maximum((hi - lo) / np.float32(maxv), np.float32(1e-8)).astype(np.float32)
    q = np.clip(np.round((wg - lo[:, :, None]) / scale[:, :, None]), 0, maxv).astype(np.uint8)
    assert np.array_equal(codes, q.reshape(16, 256))
    assert np.array_equal(S, F.bf16_trunc(scale))
    assert np.array_equal(B, F.bf16_trunc(lo))
    _, deq = orc.dequant_affine(F.pack_codes(codes, bits), S, B, 16, 256, bits)
    err = np.abs(deq.reshape(16, 4, 64) - wg)
    bound = scale[:, :, None] * 0.5 + np.abs(scale[:, :, None]) * maxv / 128 + np.abs(lo[:, :, None]) / 128
    assert np.all(err <= bound + 1e-9)


def _golden_quantizer():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "quantizer_vectors.npz")
    return np.load(path, allow_pickle=False)


@pytest.mark.parametrize("key,bits", [("pack3", 3), ("pack4", 4), ("q3", 3), ("qm4", 4), ("qm8", 8),
                                      ("qne4", 4), ("qne8", 8)])
def test_quantizer_against_reference_vectors(orc, key, bits):
    """Codes, packed bytes, scales and biases bit for bit against what the reference's own
    quantizers produced for the committed inputs (tests/golden/make_quantizer_vectors.py:
    repack_experts.quantize_affine_pack / quantize_affine_3bit, quantize_model.quantize_affine,
    quantize_non_experts.quantize_affine) — exact .5 ties, clamped scales, negative ranges."""
    g = _golden_quantizer()
    w = g["w"]
    codes, S, B = orc.quantize_affine(w, bits)
    packed = np.ascontiguousarray(F.pack_codes(codes, bits)).view(np.uint8).reshape(w.shape[0], -1)
    assert np.array_equal(packed, g[key + "_w"]), key
    assert np.array_equal(S, g[key + "_s"]) and np.array_equal(B, g[key + "_b"]), key
    # and the oracle's own packers on the same codes
    if bits == 3:
        assert np.array_equal(orc.pack_3bit(codes).reshape(w.shape[0], -1), g[key + "_w"])
    else:
        assert np.array_equal(orc.pack_u32(codes, bits).view(np.uint8).reshape(w.shape[0], -1),
                              g[key + "_w"])


def test_quantizer_vectors_hold_the_hard_cases():
    """The fixture is worth something only if it contains ties and clamped groups."""
    g = _golden_quantizer()
    w = g["w"].reshape(-1, 4, 64)
    lo, hi = w.min(2), w.max(2)
    for bits in (3, 4, 8):
        maxv = np.float32((1 << bits) - 1)
        scale = np.maximum((hi - lo) / maxv, np.float32(1e-8)).astype(np.float32)
        q = (w - lo[:, :, None]) / scale[:, :, None]
        frac = q - np.floor(q)
        assert np.count_nonzero((frac == 0.5) & (q < maxv)) >= 20, bits
    assert np.count_nonzero((hi - lo) / np.float32(7) < np.float32(1e-8)) >= 2
