"""GPU parity of the grouped chunked-prefill expert product (bf16 MFMA, pairs grouped by
expert) against the per-position CPU oracle and against the per-position GPU decode path."""
import numpy as np
import pytest

from finchmoe_amd import binding as fb
from finchmoe_amd import formats as F
from .conftest import assert_parity, cosine, rel_err

pytestmark = pytest.mark.gpu

H, I, E = 2048, 512, 12


@pytest.fixture(scope="module", params=[(3, "bf16"), (4, "bf16"), (3, "fp16"), (4, "fp16")],
                ids=["3bit", "4bit", "3bit-fp16scales", "4bit-fp16scales"])
def pstore(request):
    from finchmoe_amd import FinchHip
    bits, dtype = request.param
    sd = fb.SCALE_BF16 if dtype == "bf16" else fb.SCALE_FP16
    rng = np.random.default_rng(404)
    blob = F.synth_expert_layer(rng, E, H, I, bits, dtype)
    ctx = FinchHip(0)
    ctx.experts_config(1, E, H, I, 64, bits, sd)
    ctx.experts_upload_layer(0, blob)
    yield ctx, blob, (bits, sd)
    ctx.close()


def _routing(orc, rng, M, K, n_experts=E):
    idx = np.stack([orc.route(rng.standard_normal(n_experts).astype(np.float32), K)[0] for _ in range(M)])
    w = np.stack([orc.normalize_weights(rng.random(K).astype(np.float32)) for _ in range(M)])
    return idx.astype(np.int32), w.astype(np.float32)


@pytest.mark.parametrize("M,K", [(64, 8), (33, 8), (40, 3), (128, 8)])
def test_grouped_gemm_matches_per_position(pstore, orc, M, K):
    ctx, blob, (bits, sd) = pstore
    rng = np.random.default_rng(M * 10 + K)
    X = rng.standard_normal((M, H)).astype(np.float32)
    idx, w = _routing(orc, rng, M, K)
    out = ctx.moe_prefill(0, X, idx, w)
    worst = 0.0
    for m in range(0, M, max(1, M // 16)):       # the oracle is slow: check a spread of positions
        ref, _ = orc.moe_experts_forward(blob, X[m], idx[m], w[m], H, I, bits, scale_dtype=sd, nthreads=8)
        r, c = assert_parity(out[m], ref, "position %d" % m)
        worst = max(worst, r)
    # every position against the per-position GPU path (itself checked against the oracle)
    for m in range(M):
        single, _ = ctx.moe_decode(0, X[m], idx[m], w[m])
        assert rel_err(out[m], single) < 1e-4 and cosine(out[m], single) > 0.9999999, m
    print("M=%d K=%d worst rel err vs oracle %.2e" % (M, K, worst))
    again = ctx.moe_prefill(0, X, idx, w)
    assert np.array_equal(again, out)             # grouping order does not change results


def test_grouped_gemm_edge_inputs(pstore, orc):
    """bf16-valued activations (the benchmark's x), zero weights, out-of-range indices, all
    positions on one expert, accumulate flag."""
    import torch
    ctx, blob, (bits, sd) = pstore
    rng = np.random.default_rng(9)
    M, K = 48, 8
    X = torch.randn(M, H).to(torch.bfloat16).to(torch.float32).numpy()
    idx, w = _routing(orc, rng, M, K)
    w[5, 2] = 0.0
    idx[7, 1] = 999
    idx[9, :] = np.arange(K)                    # same experts for a run of positions
    idx[10, :] = np.arange(K)
    base = rng.standard_normal((M, H)).astype(np.float32)
    out = ctx.moe_prefill(0, X, idx, w, flags=fb.ACCUMULATE, out=base.copy())
    for m in (0, 5, 7, 9, 10, 47):
        keep = [k for k in range(K) if w[m, k] != 0 and 0 <= idx[m, k] < E]
        ref, _ = orc.moe_experts_forward(blob, X[m], idx[m, keep], w[m, keep], H, I, bits, scale_dtype=sd, nthreads=8)
        assert rel_err(out[m] - base[m], ref) < 1e-3 and cosine(out[m] - base[m], ref) > 0.99999, m


def test_small_chunks_and_guard_use_position_path(pstore, orc):
    """Below the GEMM threshold, and with FM_GUARD, the chunk equals per-position calls bitwise."""
    ctx, blob, (bits, sd) = pstore
    rng = np.random.default_rng(10)
    for M, flags in ((8, 0), (40, fb.GUARD)):
        X = rng.standard_normal((M, H)).astype(np.float32)
        idx, w = _routing(orc, rng, M, 8)
        out = ctx.moe_prefill(0, X, idx, w, flags=flags)
        for m in range(0, M, 7):
            single, _ = ctx.moe_decode(0, X[m], idx[m], w[m], flags=flags)
            assert np.array_equal(out[m], single)


@pytest.mark.parametrize("M,K", [(64, 8), (37, 5), (200, 8)])
def test_bf16_activation_entry(pstore, orc, M, K):
    """fm_moe_prefill_bf16: X as bfloat16 bits.  Contract: the fp32 entry on the widened X —
    checked against the oracle on the widened X (the parity bar) and against the fp32 entry
    (both are the same mathematics; they differ by fp32 summation order only)."""
    ctx, blob, (bits, sd) = pstore
    rng = np.random.default_rng(M + K)
    Xb = F.bf16_trunc(rng.standard_normal((M, H)).astype(np.float32))
    Xf = F.bf16_to_f32(Xb)
    idx, w = _routing(orc, rng, M, K)
    out = ctx.moe_prefill_bf16(0, Xb, idx, w)
    for m in range(0, M, max(1, M // 12)):
        ref, _ = orc.moe_experts_forward(blob, Xf[m], idx[m], w[m], H, I, bits, scale_dtype=sd, nthreads=8)
        assert_parity(out[m], ref, "bf16 entry, position %d" % m)
    wide = ctx.moe_prefill(0, Xf, idx, w)
    assert rel_err(out, wide) < 1e-4 and cosine(out, wide) > 0.9999999
    assert np.array_equal(ctx.moe_prefill_bf16(0, Xb, idx, w), out)
    # accumulate flag and an out-of-range index
    idx2 = idx.copy()
    idx2[3, 0] = -5
    base = rng.standard_normal((M, H)).astype(np.float32)
    acc = ctx.moe_prefill_bf16(0, Xb, idx2, w, flags=fb.ACCUMULATE, out=base.copy())
    plain = ctx.moe_prefill_bf16(0, Xb, idx2, w)
    assert rel_err(acc - base, plain) < 1e-5
    keep = [k for k in range(K) if 0 <= idx2[3, k] < E]
    ref, _ = orc.moe_experts_forward(blob, Xf[3], idx2[3, keep], w[3, keep], H, I, bits, scale_dtype=sd, nthreads=8)
    assert_parity(plain[3], ref, "invalid slot dropped")


def test_bf16_entry_small_chunk_is_the_position_path(pstore, orc):
    """Below the GEMM threshold the bf16 entry widens X and runs per-position decode: bitwise
    the fp32 entry on the widened X."""
    ctx, blob, (bits, sd) = pstore
    rng = np.random.default_rng(77)
    M, K = 8, 8
    Xb = F.bf16_trunc(rng.standard_normal((M, H)).astype(np.float32))
    idx, w = _routing(orc, rng, M, K)
    a = ctx.moe_prefill_bf16(0, Xb, idx, w)
    b = ctx.moe_prefill(0, F.bf16_to_f32(Xb), idx, w)
    assert np.array_equal(a, b)
