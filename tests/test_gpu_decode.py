"""GPU parity of the affine routed-expert decode path and the dequant entry points against
the CPU oracle, through the C ABI.  Bit-exact for codes and dequantized weights; GEMV outputs
within max relative error 1e-3 and cosine >= 0.99999 (fp32 accumulate)."""
import numpy as np
import pytest

from finchmoe_amd import binding as fb
from finchmoe_amd import formats as F
from .conftest import assert_parity, rel_err

pytestmark = pytest.mark.gpu

H, I = 2048, 512


@pytest.fixture(scope="module")
def store3(hip):
    """4 layers x 12 experts of synthetic 3-bit experts at the real expert shape."""
    rng = np.random.default_rng(2024)
    blobs = [F.synth_expert_layer(rng, 12, H, I, 3) for _ in range(4)]
    hip.experts_config(4, 12, H, I, 64, 3, fb.SCALE_BF16)
    for l, b in enumerate(blobs):
        hip.experts_upload_layer(l, b)
    return blobs


def _route(orc, rng, n_experts, K):
    logits = rng.standard_normal(n_experts).astype(np.float32)
    return orc.route(logits, K)


def test_dequant_bit_exact_3bit(hip, orc, store3):
    for layer, e in ((0, 0), (3, 11), (1, 5)):
        v = F.expert_views(store3[layer], e, H, I, 3)
        for which, name in ((fb.GATE, "gate"), (fb.UP, "up"), (fb.DOWN, "down")):
            W, S, B, rows, cols = v[name]
            codes, w32 = orc.dequant_affine(W, S, B, rows, cols, 3)
            gc, gw, gh = hip.dequant_expert(layer, e, which)
            assert np.array_equal(gc, codes), (layer, e, name)
            assert np.array_equal(gw.view(np.uint32), w32.view(np.uint32)), (layer, e, name)
            assert np.array_equal(gh, w32.astype(np.float16).view(np.uint16)), (layer, e, name)


def test_decode_layer_matches_oracle(hip, orc, store3):
    rng = np.random.default_rng(5)
    for layer in range(4):
        x = rng.standard_normal(H).astype(np.float32)
        idx, w = _route(orc, rng, 12, 8)
        ref, ref_eo = orc.moe_experts_forward(store3[layer], x, idx, w, H, I, 3)
        out, eo = hip.moe_decode(layer, x, idx, w)
        for k in range(8):
            assert_parity(eo[k], ref_eo[k], "layer %d slot %d" % (layer, k))
        r, c = assert_parity(out, ref, "layer %d" % layer)
        assert r < 2e-5, r   # fp32 reassociation only


def test_decode_repeatable_and_k_lt_8(hip, orc, store3):
    rng = np.random.default_rng(6)
    x = rng.standard_normal(H).astype(np.float32)
    for K in (1, 3, 8):
        idx, w = _route(orc, rng, 12, K)
        a, _ = hip.moe_decode(2, x, idx, w)
        b, _ = hip.moe_decode(2, x, idx, w)
        assert np.array_equal(a, b)    # slot-order combine: bitwise repeatable
        ref, _ = orc.moe_experts_forward(store3[2], x, idx, w, H, I, 3)
        assert_parity(a, ref, "K=%d" % K)


def test_decode_flags_and_edge_weights(hip, orc, store3):
    rng = np.random.default_rng(7)
    x = rng.standard_normal(H).astype(np.float32)
    idx = np.array([3, 9, 1, 7, 0, 11, 5, 2], np.int32)
    w = orc.normalize_weights(rng.random(8).astype(np.float32))
    ref, _ = orc.moe_experts_forward(store3[0], x, idx, w, H, I, 3)
    # accumulate: out += result
    base = rng.standard_normal(H).astype(np.float32)
    out, _ = hip.moe_decode(0, x, idx, w, flags=fb.ACCUMULATE, out=base.copy())
    assert rel_err(out, base.astype(np.float64) + ref) < 1e-5
    # weight zero and out-of-range index: the slot adds nothing
    w0 = w.copy()
    w0[2] = 0.0
    idx_bad = idx.copy()
    idx_bad[5] = 999
    ref0, _ = orc.moe_experts_forward(store3[0], x, idx[[0, 1, 3, 4, 6, 7]], w0[[0, 1, 3, 4, 6, 7]], H, I, 3)
    out0, eo0 = hip.moe_decode(0, x, idx_bad, w0)
    assert_parity(out0, ref0, "zero weight + bad index")
    assert not eo0[5].any()
    # guard flag with nothing to guard equals the plain path up to the renorm test
    outg, _ = hip.moe_decode(0, x, idx, w, flags=fb.GUARD)
    assert_parity(outg, ref, "guard")


def test_decode_guard_inf_scale(hip, orc):
    """An Inf scale in one expert: FM_GUARD drops it and renormalises like the CPU path."""
    rng = np.random.default_rng(8)
    blob = F.synth_expert_layer(rng, 4, H, I, 3)
    lo = F.expert_layout(H, I, 3)
    o = 2 * lo["expert_size"] + lo["down_s"]
    blob[o:o + 2] = np.array([0x7F80], np.uint16).view(np.uint8)
    from finchmoe_amd import FinchHip
    ctx = FinchHip(0)
    try:
        ctx.experts_config(1, 4, H, I, 64, 3, fb.SCALE_BF16)
        ctx.experts_upload_layer(0, blob)
        x = rng.standard_normal(H).astype(np.float32)
        idx = np.array([0, 2, 3], np.int32)
        w = np.array([0.5, 0.3, 0.2], np.float32)
        ref, _ = orc.moe_experts_forward(blob, x, idx, w, H, I, 3, guard=1)
        out, _ = ctx.moe_decode(0, x, idx, w, flags=fb.GUARD)
        assert np.all(np.isfinite(out))
        assert_parity(out, ref, "guarded")
        raw, _ = ctx.moe_decode(0, x, idx, w)
        assert not np.all(np.isfinite(raw))
    finally:
        ctx.close()


def test_decode_step_batched_layers(hip, orc, store3):
    """All layers in one submission == layer by layer (bitwise) == oracle (tolerance)."""
    import torch
    rng = np.random.default_rng(9)
    L, K = 4, 8
    x = rng.standard_normal((L, H)).astype(np.float32)
    idx = np.stack([_route(orc, rng, 12, K)[0] for _ in range(L)])
    w = np.stack([orc.normalize_weights(rng.random(K).astype(np.float32)) for _ in range(L)])
    dx, di, dw = (torch.from_numpy(a).cuda() for a in (x, idx, w))
    dout = torch.empty(L, H, device="cuda")
    deo = torch.empty(L, K, H, device="cuda")
    torch.cuda.synchronize()
    hip.moe_decode_step_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K,
                            dout.data_ptr(), deo.data_ptr())
    hip.sync()
    out = dout.cpu().numpy()
    for l in range(L):
        ref, ref_eo = orc.moe_experts_forward(store3[l], x[l], idx[l], w[l], H, I, 3)
        assert_parity(out[l], ref, "layer %d" % l)
        single, _ = hip.moe_decode(l, x[l], idx[l], w[l])
        assert np.array_equal(single, out[l])
        assert_parity(deo[l].cpu().numpy(), ref_eo, "expert_out layer %d" % l)


def _step_inputs(orc, seed, L, K):
    import torch
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((L, H)).astype(np.float32)
    idx = np.stack([_route(orc, rng, 12, K)[0] for _ in range(L)])
    w = np.stack([orc.normalize_weights(rng.random(K).astype(np.float32)) for _ in range(L)])
    return x, idx, w, tuple(torch.from_numpy(a).cuda() for a in (x, idx, w))


def test_fused_launch_equals_separate_kernels(hip, orc, store3):
    """One fused launch (default) == the phases as three kernels (timing mode 2), bitwise,
    also with the guard flag and with repeated launches (the two counter sets alternate)."""
    import torch
    L, K = 4, 8
    x, idx, w, (dx, di, dw) = _step_inputs(orc, 21, L, K)
    outs = {}
    for flags in (0, fb.GUARD):
        for mode in (0, 2, 0, 0):
            dout = torch.zeros(L, H, device="cuda")
            deo = torch.zeros(L, K, H, device="cuda")
            torch.cuda.synchronize()
            hip.kernel_timing(mode)
            hip.moe_decode_step_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K,
                                    dout.data_ptr(), deo.data_ptr(), flags)
            hip.sync()
            hip.kernel_timing(0)
            got = (dout.cpu().numpy(), deo.cpu().numpy())
            if flags in outs:
                assert np.array_equal(got[0], outs[flags][0]), (flags, mode)
                assert np.array_equal(got[1], outs[flags][1]), (flags, mode)
            outs[flags] = got
    ref, _ = orc.moe_experts_forward(store3[1], x[1], idx[1], w[1], H, I, 3)
    assert_parity(outs[0][0][1], ref, "fused layer 1")


def test_wait_limit_reports_instead_of_hanging(hip, orc, store3):
    """With a wait limit of zero polls the fused kernel cannot wait for other workgroups:
    it must still finish, the next sync must report the failure, and the context must work
    again afterwards."""
    import torch
    L, K = 4, 8
    x, idx, w, (dx, di, dw) = _step_inputs(orc, 22, L, K)
    dout = torch.zeros(L, H, device="cuda")
    torch.cuda.synchronize()
    hip.set_wait_limit(0)
    try:
        failed = 0
        for _ in range(20):    # a single launch can get through when every producer is early
            hip.moe_decode_step_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K,
                                    dout.data_ptr())
            try:
                hip.sync()
            except fb.FinchError as e:
                assert e.status == fb.ERR_HIP and "invalid" in str(e)
                failed += 1
        assert failed > 0
    finally:
        hip.set_wait_limit(1 << 20)
    hip.moe_decode_step_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K, dout.data_ptr())
    hip.sync()
    out = dout.cpu().numpy()
    for l in range(L):
        ref, _ = orc.moe_experts_forward(store3[l], x[l], idx[l], w[l], H, I, 3)
        assert_parity(out[l], ref, "after recovery, layer %d" % l)


@pytest.mark.parametrize("bits,dtype", [(4, "bf16"), (3, "fp16"), (4, "fp16")])
def test_other_formats(orc, bits, dtype):
    """4-bit experts and the fp16-scale variant of the benchmark text."""
    from finchmoe_amd import FinchHip
    rng = np.random.default_rng(bits * 7 + (dtype == "fp16"))
    blob = F.synth_expert_layer(rng, 9, H, I, bits, dtype)
    sd = fb.SCALE_BF16 if dtype == "bf16" else fb.SCALE_FP16
    ctx = FinchHip(0)
    try:
        ctx.experts_config(1, 9, H, I, 64, bits, sd)
        ctx.experts_upload_layer(0, blob)
        v = F.expert_views(blob, 4, H, I, bits)
        for which, name in ((fb.GATE, "gate"), (fb.DOWN, "down")):
            W, S, B, rows, cols = v[name]
            codes, w32 = orc.dequant_affine(W, S, B, rows, cols, bits, scale_dtype=sd)
            gc, gw, gh = ctx.dequant_expert(0, 4, which)
            assert np.array_equal(gc, codes)
            assert np.array_equal(gw.view(np.uint32), w32.view(np.uint32))
            assert np.array_equal(gh, w32.astype(np.float16).view(np.uint16))
        x = rng.standard_normal(H).astype(np.float32)
        idx, w = _route(orc, rng, 9, 8)
        ref, ref_eo = orc.moe_experts_forward(blob, x, idx, w, H, I, bits, scale_dtype=sd)
        out, eo = ctx.moe_decode(0, x, idx, w)
        assert_parity(eo, ref_eo, "expert_out")
        assert_parity(out, ref, "moe_out")
    finally:
        ctx.close()


def test_other_shape_397b_class(orc):
    """hidden 4096 / inter 1024 (the sibling model's expert shape, repack_experts.py:108-119)."""
    from finchmoe_amd import FinchHip
    rng = np.random.default_rng(31)
    h, i = 4096, 1024
    blob = F.synth_expert_layer(rng, 3, h, i, 4)
    ctx = FinchHip(0)
    try:
        ctx.experts_config(1, 3, h, i, 64, 4, fb.SCALE_BF16)
        ctx.experts_upload_layer(0, blob)
        x = rng.standard_normal(h).astype(np.float32)
        idx = np.array([2, 0], np.int32)
        w = np.array([0.25, 0.75], np.float32)
        ref, _ = orc.moe_experts_forward(blob, x, idx, w, h, i, 4)
        out, _ = ctx.moe_decode(0, x, idx, w)
        assert_parity(out, ref, "4096/1024")
    finally:
        ctx.close()


@pytest.mark.parametrize("h,i,bits", [(1024, 256, 3), (512, 128, 3), (1024, 512, 4), (512, 256, 4)])
def test_small_shapes_cover_every_lane_map(orc, h, i, bits):
    """hidden/inter combinations that exercise 8/4 lanes per gate row and 2/1/4 lanes per
    down row (the kernels are specialised on lanes-per-row)."""
    from finchmoe_amd import FinchHip
    rng = np.random.default_rng(h + i + bits)
    blob = F.synth_expert_layer(rng, 5, h, i, bits)
    ctx = FinchHip(0)
    try:
        ctx.experts_config(1, 5, h, i, 64, bits, fb.SCALE_BF16)
        ctx.experts_upload_layer(0, blob)
        x = rng.standard_normal(h).astype(np.float32)
        idx = np.array([4, 0, 2], np.int32)
        w = np.array([0.5, 0.2, 0.3], np.float32)
        ref, ref_eo = orc.moe_experts_forward(blob, x, idx, w, h, i, bits)
        out, eo = ctx.moe_decode(0, x, idx, w)
        assert_parity(eo, ref_eo, "expert_out %d/%d" % (h, i))
        assert_parity(out, ref, "moe_out %d/%d" % (h, i))
    finally:
        ctx.close()


def test_prefill_small_chunk_equals_per_position(hip, orc, store3):
    """Chunk of 8 positions (the reference default, infer.m:455): identical to running the
    decode call per position — bitwise, as the reference's bench_prefill.sh demands."""
    rng = np.random.default_rng(10)
    M, K = 8, 8
    X = rng.standard_normal((M, H)).astype(np.float32)
    idx = np.stack([_route(orc, rng, 12, K)[0] for _ in range(M)])
    w = np.stack([orc.normalize_weights(rng.random(K).astype(np.float32)) for _ in range(M)])
    out = hip.moe_prefill(1, X, idx, w)
    for m in range(M):
        single, _ = hip.moe_decode(1, X[m], idx[m], w[m])
        assert np.array_equal(out[m], single), m
        ref, _ = orc.moe_experts_forward(store3[1], X[m], idx[m], w[m], H, I, 3)
        assert_parity(out[m], ref, "position %d" % m)


def test_errors_are_codes_not_aborts(hip, store3):
    x = np.zeros(H, np.float32)
    idx = np.arange(8, dtype=np.int32)
    w = np.full(8, 0.125, np.float32)
    from finchmoe_amd import FinchError
    with pytest.raises(FinchError) as e:
        hip.moe_decode(99, x, idx, w)
    assert e.value.status == fb.ERR_ARG
    with pytest.raises(FinchError):
        hip.experts_upload_layer(0, np.zeros(100, np.uint8))
    L = hip.L
    assert L.fm_moe_decode(hip.h, 0, x.ctypes.data, idx.ctypes.data, w.ctypes.data, 9,
                           x.ctypes.data, None, 0) == fb.ERR_ARG
    from finchmoe_amd import FinchHip
    c2 = FinchHip(0)
    try:
        with pytest.raises(FinchError) as e:
            c2.hidden = H
            c2.moe_decode(0, x, idx, w)
        assert e.value.status == fb.ERR_STATE
        with pytest.raises(FinchError) as e:
            c2.experts_config(1, 4, 2048, 512, 32, 3, 0)
        assert e.value.status == fb.ERR_UNSUPPORTED
        c2.experts_config(2, 4, H, I, 64, 3, 0)
        with pytest.raises(FinchError) as e:
            c2.moe_decode(1, x, idx, w)     # configured, layer never uploaded
        assert e.value.status == fb.ERR_STATE
    finally:
        c2.close()


def test_host_call_falls_back_to_separate_kernels(hip, orc, store3):
    """With a wait limit of zero polls the one-launch kernel gives up on its waits; the
    synchronous entry point then repeats the call as separate kernels and still returns the
    right result."""
    rng = np.random.default_rng(23)
    x = rng.standard_normal(H).astype(np.float32)
    idx, w = _route(orc, rng, 12, 8)
    ref, ref_eo = orc.moe_experts_forward(store3[1], x, idx, w, H, I, 3)
    hip.set_wait_limit(0)
    try:
        for _ in range(8):
            out, eo = hip.moe_decode(1, x, idx, w)
            assert_parity(out, ref, "fallback result")
            assert_parity(eo, ref_eo, "fallback expert outputs")
    finally:
        hip.set_wait_limit(1 << 20)


def test_row_sum_launch_equals_counter_launch(hip, orc, store3):
    """Without a buffer for the per-expert vectors the operator takes the launch that sums the
    experts in LDS: its result equals, bit for bit, the launch that writes the per-expert
    vectors and combines them — for steps of different sizes in a row (the two activation
    sets alternate and re-mark what the launch before filled), with the accumulate flag, with
    K below 8, and with an expert index out of range."""
    import torch
    for seed, L, K, flags in ((31, 4, 8, 0), (32, 1, 8, 0), (33, 3, 8, fb.ACCUMULATE), (34, 4, 4, 0),
                              (35, 2, 8, 0), (36, 4, 3, 0), (37, 4, 8, 0), (38, 1, 1, fb.ACCUMULATE)):
        x, idx, w, (dx, di, dw) = _step_inputs(orc, seed, L, K)
        if seed == 37:
            idx[2, 5] = 99                                  # out of range: contributes zero
            di = torch.from_numpy(idx).cuda()
        base = torch.from_numpy(np.random.default_rng(seed).standard_normal((L, H)).astype(np.float32)).cuda()
        want = base.clone()
        deo = torch.zeros(L, K, H, device="cuda")
        torch.cuda.synchronize()
        hip.moe_decode_step_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K,
                                want.data_ptr(), deo.data_ptr(), flags)
        hip.sync()
        for rep in range(2):
            got = base.clone()
            torch.cuda.synchronize()
            hip.moe_decode_step_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K,
                                    got.data_ptr(), None, flags)
            hip.sync()
            assert torch.equal(got, want), (seed, L, K, flags, rep)
        l = L - 1
        keep = (idx[l] >= 0) & (idx[l] < 12)
        ref, _ = orc.moe_experts_forward(store3[l], x[l], idx[l][keep], w[l][keep], H, I, 3)
        mine = want[l].cpu().numpy() - (base[l].cpu().numpy() if flags & fb.ACCUMULATE else 0)
        assert rel_err(mine, ref) < 1e-3, (seed, rel_err(mine, ref))


@pytest.mark.parametrize("h,i,bits,dtype", [(1024, 256, 3, "bf16"), (512, 128, 3, "bf16"), (1024, 256, 4, "fp16"),
                                            (512, 128, 4, "bf16"), (2048, 512, 4, "bf16"), (2048, 512, 3, "fp16")])
def test_row_sum_launch_other_shapes(orc, h, i, bits, dtype):
    """The same equality where the lane maps differ (16/8/4 lanes per gate row, 4/2/1 per down
    row), for 4-bit codes and FP16 scales, on a step of several layers."""
    import torch
    from finchmoe_amd import FinchHip
    rng = np.random.default_rng(h + i + bits)
    L, E, K = 3, 6, 4
    blobs = [F.synth_expert_layer(rng, E, h, i, bits, dtype) for _ in range(L)]
    ctx = FinchHip(0)
    try:
        sd = fb.SCALE_FP16 if dtype == "fp16" else fb.SCALE_BF16
        ctx.experts_config(L, E, h, i, 64, bits, sd)
        for l, b in enumerate(blobs):
            ctx.experts_upload_layer(l, b)
        x = rng.standard_normal((L, h)).astype(np.float32)
        idx = np.stack([rng.permutation(E)[:K] for _ in range(L)]).astype(np.int32)
        w = rng.random((L, K)).astype(np.float32)
        dx, di, dw = (torch.from_numpy(a).cuda() for a in (x, idx, w))
        want, got = torch.zeros(L, h, device="cuda"), torch.zeros(L, h, device="cuda")
        deo = torch.zeros(L, K, h, device="cuda")
        torch.cuda.synchronize()
        ctx.moe_decode_step_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K, want.data_ptr(), deo.data_ptr(), 0)
        ctx.moe_decode_step_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K, got.data_ptr(), None, 0)
        ctx.sync()
        assert torch.equal(got, want)
        ref, _ = orc.moe_experts_forward(blobs[1], x[1], idx[1], w[1], h, i, bits, scale_dtype=sd)
        assert_parity(got[1].cpu().numpy(), ref, "layer 1 %d/%d/%d" % (h, i, bits))
    finally:
        ctx.close()
