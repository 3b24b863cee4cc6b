"""Pins of the CPU oracle's matvec, activation, routing and expert-block code (no GPU):
float64 recomputation from independently dequantized weights, special cases that reduce to
closed forms, brute force on small routing inputs, failure injection."""
import itertools

import numpy as np
import pytest

from finchmoe_amd import formats as F
from .conftest import cosine, rel_err


def _dequant64(codes, S, B, dtype="bf16"):
    if dtype == "bf16":
        s, b = F.bf16_to_f32(S).astype(np.float64), F.bf16_to_f32(B).astype(np.float64)
    else:
        s, b = S.view(np.float16).astype(np.float64), B.view(np.float16).astype(np.float64)
    g = np.arange(codes.shape[1]) // 64
    return codes.astype(np.float64) * s[:, g] + b[:, g]


@pytest.mark.parametrize("bits", [3, 4, 8])
def test_matvec_vs_float64(orc, bits):
    rng = np.random.default_rng(bits)
    out_dim, in_dim = 96, 1024
    codes, W, S, B = F.synth_affine_tensor(rng, out_dim, in_dim, bits)
    x = rng.standard_normal(in_dim).astype(np.float32)
    got = orc.dequant_matvec(W, S, B, x, out_dim, in_dim, bits)
    want = _dequant64(codes, S, B) @ x.astype(np.float64)
    assert rel_err(got, want) < 2e-5 and cosine(got, want) > 0.9999999
    # rows split over threads: per-row arithmetic unchanged -> bit identical
    mt = orc.dequant_matvec(W, S, B, x, out_dim, in_dim, bits, nthreads=5)
    assert np.array_equal(mt.view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("bits", [3, 4])
def test_matvec_special_cases(orc, bits):
    rng = np.random.default_rng(40 + bits)
    out_dim, in_dim = 32, 512
    codes, W, S, B = F.synth_affine_tensor(rng, out_dim, in_dim, bits)
    x = rng.standard_normal(in_dim).astype(np.float32)
    # scale = 0  =>  out = sum_g bias_g * sum(x in g) (codes drop out entirely)
    S0 = np.zeros_like(S)
    ones = np.ones(in_dim, np.float32)
    got = orc.dequant_matvec(W, S0, B, ones, out_dim, in_dim, bits)
    want = (F.bf16_to_f32(B).astype(np.float64) * 64.0).sum(1)
    assert rel_err(got, want) < 1e-5
    # one-hot x  =>  out = one dequantized column, bit exact (ties matvec to dequant)
    _, wf = orc.dequant_affine(W, S, B, out_dim, in_dim, bits)
    for col in (0, 7, 8, 63, 64, 65, 200, in_dim - 1):
        e = np.zeros(in_dim, np.float32)
        e[col] = 1.0
        got = orc.dequant_matvec(W, S, B, e, out_dim, in_dim, bits)
        assert np.array_equal(got.view(np.uint32), (wf[:, col] + np.float32(0)).view(np.uint32)), col
    # linearity in x (fp32 tolerance)
    y = rng.standard_normal(in_dim).astype(np.float32)
    a = orc.dequant_matvec(W, S, B, x, out_dim, in_dim, bits)
    b = orc.dequant_matvec(W, S, B, y, out_dim, in_dim, bits)
    ab = orc.dequant_matvec(W, S, B, x + y, out_dim, in_dim, bits)
    assert rel_err(ab, a.astype(np.float64) + b) < 1e-5


@pytest.mark.parametrize("gtype,bits", [(12, 10), (14, 11)])
def test_gguf_matvec_vs_float64(orc, gtype, bits):
    rng = np.random.default_rng(gtype)
    out_dim, in_dim = 40, 1024
    W = F.synth_gguf_tensor(rng, out_dim, in_dim, gtype)
    x = rng.standard_normal(in_dim).astype(np.float32)
    got = orc.dequant_matvec(W, None, None, x, out_dim, in_dim, bits)
    want = orc.gguf_dequant(W, out_dim, in_dim, gtype).astype(np.float64) @ x.astype(np.float64)
    assert rel_err(got, want) < 2e-5 and cosine(got, want) > 0.9999999


def test_swiglu(orc):
    rng = np.random.default_rng(3)
    g = (rng.standard_normal(4096) * 4).astype(np.float32)
    u = rng.standard_normal(4096).astype(np.float32)
    got = orc.swiglu(g, u)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = g64 / (1 + np.exp(-g64)) * u64
    assert np.max(np.abs(got - want)) < 1e-5
    assert orc.swiglu(np.zeros(4, np.float32), np.ones(4, np.float32)).tolist() == [0, 0, 0, 0]
    big = orc.swiglu(np.array([50.0, -50.0], np.float32), np.array([2.0, 2.0], np.float32))
    assert big[0] == 100.0 and abs(big[1]) < 1e-18


def test_softmax_topk_normalise(orc):
    rng = np.random.default_rng(4)
    for n, K in ((16, 4), (256, 8), (9, 8), (8, 8)):
        logits = rng.standard_normal(n).astype(np.float32)
        p = orc.softmax(logits)
        p64 = np.exp(logits.astype(np.float64) - logits.max())
        p64 /= p64.sum()
        assert np.allclose(p, p64, rtol=1e-5, atol=1e-9) and abs(p.sum() - 1) < 1e-5
        idx, val = orc.topk(p, K)
        assert len(set(idx.tolist())) == K
        assert set(idx.tolist()) == set(np.argsort(-p, kind="stable")[:K].tolist())
        assert np.array_equal(val, p[idx])
        w = orc.normalize_weights(val)
        assert abs(w.sum() - 1) < 1e-6 and np.allclose(w, val / val.sum(), rtol=1e-6)


def _topk_model(scores, K):
    """Straight python model of the slot-replacement rule (infer.m:1811-1830)."""
    vals, idx = [-1e30] * K, [0] * K
    for i, s in enumerate(scores):
        mn = min(range(K), key=lambda k: (vals[k], k))
        if s > vals[mn]:
            vals[mn], idx[mn] = s, i
    return idx, vals


def test_topk_brute_force_and_ties(orc):
    """All orderings of small inputs with repeated values: slot order is part of the
    contract (weights are summed in slot order)."""
    base = [0.5, 0.25, 0.25, 0.125, 0.75]
    for perm in itertools.permutations(base):
        s = np.array(perm, np.float32)
        for K in (1, 2, 3):
            idx, val = orc.topk(s, K)
            mi, mv = _topk_model(list(perm), K)
            assert idx.tolist() == mi and val.tolist() == [np.float32(v) for v in mv]
    # ties keep the earlier index
    idx, _ = orc.topk(np.array([1, 1, 1, 1], np.float32), 2)
    assert idx.tolist() == [0, 1]
    # weights all zero: normalise leaves them
    assert orc.normalize_weights(np.zeros(4, np.float32)).tolist() == [0, 0, 0, 0]


@pytest.mark.parametrize("bits", [3, 4])
def test_expert_block_vs_float64(orc, bits):
    rng = np.random.default_rng(100 + bits)
    H, I, E, K = 512, 256, 6, 4
    blob = F.synth_expert_layer(rng, E, H, I, bits)
    x = rng.standard_normal(H).astype(np.float32)
    idx = np.array([4, 1, 5, 0], np.int32)
    w = orc.normalize_weights(rng.random(K).astype(np.float32))
    moe, eo, g, u, a = orc.moe_experts_forward(blob, x, idx, w, H, I, bits, stages=True)
    want = np.zeros(H)
    for k in range(K):
        v = F.expert_views(blob, int(idx[k]), H, I, bits)
        mats = {}
        for name in ("gate", "up", "down"):
            W, S, B, rows, cols = v[name]
            codes, _ = orc.dequant_affine(W, S, B, rows, cols, bits)
            mats[name] = _dequant64(codes, S, B)
        g64 = mats["gate"] @ x.astype(np.float64)
        u64 = mats["up"] @ x.astype(np.float64)
        a64 = g64 / (1 + np.exp(-g64)) * u64
        o64 = mats["down"] @ a64
        assert rel_err(g[k], g64) < 2e-5 and rel_err(u[k], u64) < 2e-5
        assert rel_err(a[k], a64) < 5e-5 and rel_err(eo[k], o64) < 1e-4
        want += float(w[k]) * o64
    assert rel_err(moe, want) < 1e-4 and cosine(moe, want) > 0.999999
    # guard on, nothing to guard: same numbers
    moe_g, _ = orc.moe_experts_forward(blob, x, idx, w, H, I, bits, guard=1)
    assert np.array_equal(moe_g, moe)
    # slot order matters only through fp32 association; permuting slots permutes eo
    perm = np.array([2, 0, 3, 1])
    moe_p, eo_p = orc.moe_experts_forward(blob, x, idx[perm], w[perm], H, I, bits)
    assert np.array_equal(eo_p, eo[perm]) and rel_err(moe_p, moe) < 1e-5


def test_expert_block_guard_and_zero_weight(orc):
    """Inf scale in one expert: guard=1 drops it and renormalises (infer.m:10190-10204);
    guard=0 propagates it; w=0 leaves the other experts' sum."""
    rng = np.random.default_rng(7)
    H, I, E, K, bits = 512, 256, 4, 3, 3
    blob = F.synth_expert_layer(rng, E, H, I, bits)
    lo = F.expert_layout(H, I, bits)
    bad = blob.copy()
    o = 2 * lo["expert_size"] + lo["down_s"]
    bad[o:o + 2] = np.array([0x7F80], np.uint16).view(np.uint8)   # +Inf bf16 scale
    x = rng.standard_normal(H).astype(np.float32)
    idx = np.array([0, 2, 3], np.int32)
    w = np.array([0.5, 0.3, 0.2], np.float32)
    moe_raw, eo = orc.moe_experts_forward(bad, x, idx, w, H, I, bits, guard=0)
    assert not np.all(np.isfinite(moe_raw)) and not np.all(np.isfinite(eo[1]))
    moe_g, _ = orc.moe_experts_forward(bad, x, idx, w, H, I, bits, guard=1)
    assert np.all(np.isfinite(moe_g))
    keep, _ = orc.moe_experts_forward(blob, x, idx[[0, 2]], w[[0, 2]], H, I, bits, guard=0)
    assert rel_err(moe_g, keep / np.float32(0.7)) < 1e-6      # renormalised by 1/(0.5+0.2)
    # weight zero: slot contributes nothing
    w0 = np.array([0.6, 0.0, 0.4], np.float32)
    a, _ = orc.moe_experts_forward(blob, x, idx, w0, H, I, bits)
    b, _ = orc.moe_experts_forward(blob, x, idx[[0, 2]], w0[[0, 2]], H, I, bits)
    assert np.array_equal(a, b)
    # accumulation into moe_out is += : K=0 leaves it untouched
    z, _ = orc.moe_experts_forward(blob, x, idx[:0], w[:0], H, I, bits)
    assert not z.any()


def test_gguf_expert_block_vs_float64(orc):
    rng = np.random.default_rng(11)
    H, I, E = 512, 256, 3
    gate, up, down = F.synth_gguf_layer(rng, E, H, I)
    x = rng.standard_normal(H).astype(np.float32)
    idx = np.array([2, 0], np.int32)
    w = np.array([0.7, 0.3], np.float32)
    moe, eo = orc.moe_gguf_forward(gate, up, down, x, idx, w, H, I)
    G = orc.gguf_dequant(gate, E * I, H, 12).astype(np.float64).reshape(E, I, H)
    U = orc.gguf_dequant(up, E * I, H, 12).astype(np.float64).reshape(E, I, H)
    D = orc.gguf_dequant(down, E * H, I, 14).astype(np.float64).reshape(E, H, I)
    want = np.zeros(H)
    for k, e in enumerate(idx):
        g64, u64 = G[e] @ x.astype(np.float64), U[e] @ x.astype(np.float64)
        o64 = D[e] @ (g64 / (1 + np.exp(-g64)) * u64)
        assert rel_err(eo[k], o64) < 1e-4
        want += float(w[k]) * o64
    assert rel_err(moe, want) < 1e-4


def test_bf16_operand_model_bound(orc):
    """The bf16-operand model (what an MFMA GEMM may do) stays inside the parity bar of the
    fp32 path on the benchmark's weight distribution — checked before relying on it."""
    rng = np.random.default_rng(12)
    out_dim, in_dim = 128, 2048
    codes, W, S, B = F.synth_affine_tensor(rng, out_dim, in_dim, 3)
    x = rng.standard_normal(in_dim).astype(np.float32)
    a = orc.dequant_matvec(W, S, B, x, out_dim, in_dim, 3)
    b = orc.dequant_matvec_bf16model(W, S, B, x, out_dim, in_dim, 3)
    print("bf16 model vs fp32 path: rel_err %.3e cosine %.8f" % (rel_err(b, a), cosine(b, a)))
    assert cosine(b, a) > 0.9999


def test_layer_tail_against_float64_and_special_cases(orc):
    """orc_layer_tail (infer.m:9608-9760, shaders.metal:2196-2231, 1134-1205) against a float64
    evaluation built from the dequantized weights, and the cases that pin each term: zero
    expert weights drop the expert sum, a very negative gate score drops the shared expert,
    the norm of c*x equals the norm of x for eps -> 0."""
    from finchmoe_amd import formats as F
    rng = np.random.default_rng(21)
    hidden, si, K = 256, 128, 4
    codes, W, S, B = F.synth_affine_tensor(rng, hidden, si, 4, "bf16")
    wd = orc.dequant_affine(W, S, B, hidden, si, 4)[1].astype(np.float64)
    h_mid = rng.standard_normal(hidden).astype(np.float32)
    eo = rng.standard_normal((K, hidden)).astype(np.float32)
    params = np.zeros(10, np.float32)
    params[:K] = [0.4, 0.3, 0.2, 0.1]
    params[8] = 0.7
    sg = rng.standard_normal(si).astype(np.float32)
    su = rng.standard_normal(si).astype(np.float32)
    nw = ((1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    hid, nxt = orc.layer_tail(W, S, B, h_mid, eo, params, K, sg, su, nw)
    g = sg.astype(np.float64)
    act = g / (1 + np.exp(-g)) * su
    want = h_mid + (params[:K, None].astype(np.float64) * eo).sum(0) + wd @ act / (1 + np.exp(-0.7))
    assert np.abs(hid - want).max() < 1e-5 * np.abs(want).max()
    wn = (nw.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    want_n = want / np.sqrt(np.mean(want ** 2) + 1e-6) * wn
    assert np.abs(nxt - want_n).max() < 1e-5 * np.abs(want_n).max()
    # special cases
    p0 = params.copy()
    p0[:K] = 0
    p0[8] = -200.0
    hid0, _ = orc.layer_tail(W, S, B, h_mid, eo, p0, K, sg, su, None)
    assert np.array_equal(hid0, h_mid)
    a = orc.rms_norm(h_mid, nw, 0.0)
    b = orc.rms_norm(3.0 * h_mid, nw, 0.0)
    assert np.abs(a - b).max() < 1e-6
    ones = np.full(hidden, 0x3F80, np.uint16)
    assert abs(float(np.mean(orc.rms_norm(h_mid, ones, 0.0).astype(np.float64) ** 2)) - 1.0) < 1e-6
