"""Pins the CPU oracle (oracle/fm_oracle.c) against the reference's own C text, compiled by
oracle/build_ref.sh into oracle/_ref/libfm_ref.so from finchmoe/infer.m:686-702, 1575-1881.
Every comparison is bit for bit: both sides are plain fp32 C compiled with the same flags, and
the restatement keeps the reference's evaluation order.  No GPU."""
import ctypes as C

import numpy as np
import pytest

from finchmoe_amd import formats as F


@pytest.fixture(scope="module")
def ref(orc):
    R = orc.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref/libfm_ref.so not built (needs the reference tree: make -C oracle ref)")
    return R


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def test_widening_exhaustive(orc, ref):
    L = orc.lib()
    for h in range(65536):
        a, b = L.orc_fp16_to_f32(h), ref.ref_fp16_to_f32(h)
        assert (a != a and b != b) or np.float32(a).view(np.uint32) == np.float32(b).view(np.uint32), h
        a, b = L.orc_bf16_to_f32(h), ref.ref_bf16_to_f32(h)
        assert (a != a and b != b) or np.float32(a).view(np.uint32) == np.float32(b).view(np.uint32), h
    rng = np.random.default_rng(0)
    for v in rng.standard_normal(2000).astype(np.float32) * np.float32(37.0):
        assert L.orc_f32_to_bf16_trunc(float(v)) == ref.ref_f32_to_bf16(float(v))


def test_scale_min_k4_random_bytes(orc, ref):
    """All 8 sub-blocks over random 12-byte fields: pins which byte supplies the high two
    bits for j >= 4 (a swap of scales[j-4] / scales[j] changes the output)."""
    L = orc.lib()
    rng = np.random.default_rng(1)
    sc = (C.c_uint8 * 1)()
    m = (C.c_uint8 * 1)()
    sc2 = (C.c_uint8 * 1)()
    m2 = (C.c_uint8 * 1)()
    for _ in range(2000):
        s = rng.integers(0, 256, 12, dtype=np.uint8)
        for j in range(8):
            L.orc_get_scale_min_k4(j, s.ctypes.data, sc, m)
            ref.ref_get_scale_min_k4(j, s.ctypes.data, sc2, m2)
            assert (sc[0], m[0]) == (sc2[0], m2[0]), (j, s)


@pytest.mark.parametrize("ggml_type", [12, 14])
def test_gguf_dequant_row(orc, ref, ggml_type):
    L = orc.lib()
    rng = np.random.default_rng(ggml_type)
    in_dim = 1024
    W = F.synth_gguf_tensor(rng, 6, in_dim, ggml_type)
    rb = F.gguf_row_bytes(in_dim, ggml_type)
    a = np.empty(in_dim, np.float32)
    b = np.empty(in_dim, np.float32)
    for r in range(6):
        L.orc_gguf_dequant_row(W.ctypes.data + r * rb, a.ctypes.data, in_dim, ggml_type)
        ref.ref_gguf_dequant_row(W.ctypes.data + r * rb, b.ctypes.data, in_dim, ggml_type)
        assert np.array_equal(_bits(a), _bits(b)), r


@pytest.mark.parametrize("bits", [3, 4, 8])
def test_matvec_affine(orc, ref, bits):
    rng = np.random.default_rng(100 + bits)
    out_dim, in_dim = 48, 1024
    _, W, S, B = F.synth_affine_tensor(rng, out_dim, in_dim, bits)
    x = rng.standard_normal(in_dim).astype(np.float32)
    got = orc.dequant_matvec(W, S, B, x, out_dim, in_dim, bits)
    want = np.empty(out_dim, np.float32)
    ref.ref_cpu_dequant_matvec(W.ctypes.data, S.ctypes.data, B.ctypes.data, x.ctypes.data,
                               want.ctypes.data, out_dim, in_dim, 64, bits)
    assert np.array_equal(_bits(got), _bits(want))


@pytest.mark.parametrize("bits,ggml_type", [(10, 12), (11, 14)])
def test_matvec_gguf(orc, ref, bits, ggml_type):
    rng = np.random.default_rng(bits)
    out_dim, in_dim = 24, 512
    W = F.synth_gguf_tensor(rng, out_dim, in_dim, ggml_type)
    x = rng.standard_normal(in_dim).astype(np.float32)
    got = orc.dequant_matvec(W, None, None, x, out_dim, in_dim, bits)
    want = np.empty(out_dim, np.float32)
    ref.ref_cpu_dequant_matvec(W.ctypes.data, None, None, x.ctypes.data, want.ctypes.data,
                               out_dim, in_dim, 64, bits)
    assert np.array_equal(_bits(got), _bits(want))


def test_matvec_raw_bf16(orc, ref):
    """scales == NULL and bits not 10/11: W is unquantized BF16 [out][in]."""
    rng = np.random.default_rng(7)
    out_dim, in_dim = 40, 768
    W = F.bf16_trunc(rng.standard_normal((out_dim, in_dim)).astype(np.float32))
    x = rng.standard_normal(in_dim).astype(np.float32)
    for bits in (4, 16, 0):
        got = orc.dequant_matvec(W, None, None, x, out_dim, in_dim, bits)
        want = np.empty(out_dim, np.float32)
        ref.ref_cpu_dequant_matvec(W.ctypes.data, None, None, x.ctypes.data, want.ctypes.data,
                                   out_dim, in_dim, 64, bits)
        assert np.array_equal(_bits(got), _bits(want)), bits
    # and it is what the mathematics says (float64 from the widened weights)
    w64 = F.bf16_to_f32(W).astype(np.float64)
    assert np.max(np.abs(got - w64 @ x)) < 1e-3


def test_routing_and_activation(orc, ref):
    rng = np.random.default_rng(3)
    for trial in range(50):
        n = int(rng.integers(8, 300))
        K = int(rng.integers(1, 9))
        logits = rng.standard_normal(n).astype(np.float32)
        if trial % 5 == 0:                       # ties exercise the slot rule
            logits = np.round(logits * 2) / 2
        logits = logits.astype(np.float32)
        p = orc.softmax(logits)
        q = logits.copy()
        ref.ref_cpu_softmax(q.ctypes.data, n)
        assert np.array_equal(_bits(p), _bits(q))
        idx, val = orc.topk(p, K)
        idx2 = np.empty(K, np.int32)
        val2 = np.empty(K, np.float32)
        ref.ref_cpu_topk(q.ctypes.data, n, K, idx2.ctypes.data, val2.ctypes.data)
        assert np.array_equal(idx, idx2) and np.array_equal(_bits(val), _bits(val2))
        w = orc.normalize_weights(val)
        ref.ref_cpu_normalize_weights(val2.ctypes.data, K)
        assert np.array_equal(_bits(w), _bits(val2))
    g = rng.standard_normal(512).astype(np.float32) * 4
    u = rng.standard_normal(512).astype(np.float32)
    a = orc.swiglu(g, u)
    b = np.empty(512, np.float32)
    ref.ref_cpu_swiglu(g.ctypes.data, u.ctypes.data, b.ctypes.data, 512)
    assert np.array_equal(_bits(a), _bits(b))


def test_rms_norm_and_madd(orc, ref):
    rng = np.random.default_rng(4)
    x = rng.standard_normal(2048).astype(np.float32)
    w = F.bf16_trunc(1.0 + 0.1 * rng.standard_normal(2048).astype(np.float32))
    a = orc.rms_norm(x, w, 1e-6)
    b = np.empty(2048, np.float32)
    ref.ref_cpu_rms_norm(x.ctypes.data, w.ctypes.data, b.ctypes.data, 2048, 1e-6)
    assert np.array_equal(_bits(a), _bits(b))
    L = orc.lib()
    d1 = rng.standard_normal(2048).astype(np.float32)
    d2 = d1.copy()
    L.orc_vec_madd(d1.ctypes.data, x.ctypes.data, 0.37, 2048)
    ref.ref_cpu_vec_madd(d2.ctypes.data, x.ctypes.data, 0.37, 2048)
    assert np.array_equal(_bits(d1), _bits(d2))
