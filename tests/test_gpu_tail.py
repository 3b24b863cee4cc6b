"""GPU parity of the layer tail (shared expert down projection, combine with residual, next
layer's RMS norm) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from finchmoe_amd import binding as fb
from finchmoe_amd import formats as F
from .conftest import assert_parity, rel_err

pytestmark = pytest.mark.gpu


def _bf16(x):
    return (np.ascontiguousarray(x, np.float32).view(np.uint32) >> 16).astype(np.uint16)


def _run(hip, orc, rng, hidden, si, bits, K, dtype="bf16", with_norm=True, score=0.3):
    import torch
    codes, W, S, B = F.synth_affine_tensor(rng, hidden, si, bits, dtype)
    sd = fb.SCALE_BF16 if dtype == "bf16" else fb.SCALE_FP16
    t = hip.tensor_register(W, S, B, hidden, si, bits, 64, sd)
    h_mid = rng.standard_normal(hidden).astype(np.float32)
    eo = (rng.standard_normal((max(K, 1), hidden)) * 3).astype(np.float32)
    params = np.zeros(10, np.float32)
    params[:K] = orc.normalize_weights(rng.random(max(K, 1)).astype(np.float32))[:K]
    params[8] = score
    sg = rng.standard_normal(si).astype(np.float32)
    su = rng.standard_normal(si).astype(np.float32)
    nw = _bf16(1.0 + 0.1 * rng.standard_normal(hidden))
    ref_h, ref_n = orc.layer_tail(W, S, B, h_mid, eo, params, K, sg, su, nw if with_norm else None,
                                  bits=bits, scale_dtype=sd)
    dev = [torch.from_numpy(a).cuda() for a in (h_mid, eo, params, sg, su)]
    d_nw = torch.from_numpy(nw.view(np.int16)).cuda()
    d_hid = torch.zeros(hidden, device="cuda")
    d_next = torch.zeros(hidden, device="cuda")
    torch.cuda.synchronize()
    outs = []
    for _ in range(3):      # the ticket counter must come back to zero every time
        d_hid.zero_()
        d_next.zero_()
        torch.cuda.synchronize()
        hip.layer_tail_dev(t, dev[0].data_ptr(), dev[1].data_ptr() if K else None, dev[2].data_ptr(), K,
                           dev[3].data_ptr(), dev[4].data_ptr(),
                           d_nw.data_ptr() if with_norm else None, 1e-6, d_hid.data_ptr(),
                           d_next.data_ptr() if with_norm else None)
        hip.sync()
        outs.append((d_hid.cpu().numpy(), d_next.cpu().numpy()))
    hip.tensor_release(t)
    for h, n in outs:
        assert_parity(h, ref_h, "hidden")
        assert rel_err(h, ref_h) < 2e-5
        if with_norm:
            assert_parity(n, ref_n, "next input")
            assert rel_err(n, ref_n) < 2e-5
        else:
            assert not n.any()
        assert np.array_equal(h, outs[0][0]) and np.array_equal(n, outs[0][1])
    return outs[0], (ref_h, ref_n), (h_mid, eo, params, nw)


def test_layer_tail_reference_shape(hip, orc):
    """hidden 2048, shared intermediate 512, 4-bit, K = 8 (infer.m:150-154)."""
    _run(hip, orc, np.random.default_rng(1), 2048, 512, 4, 8)


@pytest.mark.parametrize("hidden,si,bits,K,dtype", [(1024, 128, 4, 3, "bf16"), (4096, 256, 3, 8, "fp16"),
                                                    (2048, 1024, 8, 1, "bf16"), (512, 2048, 4, 0, "bf16")])
def test_layer_tail_shapes(hip, orc, hidden, si, bits, K, dtype):
    _run(hip, orc, np.random.default_rng(hidden + si), hidden, si, bits, K, dtype)


def test_layer_tail_last_layer_and_closed_forms(hip, orc):
    """No next layer: only hidden is written.  With K = 0 and a shared gate score of -inf-like
    size the result is h_mid itself; the norm of a vector equals the library formula."""
    rng = np.random.default_rng(5)
    _run(hip, orc, rng, 2048, 512, 4, 8, with_norm=False)
    (h, n), _, (h_mid, eo, params, nw) = _run(hip, orc, rng, 2048, 512, 4, 0, score=-200.0)
    assert np.array_equal(h, h_mid)
    w = (nw.astype(np.uint32) << 16).view(np.float32)
    want = h_mid.astype(np.float64) / np.sqrt(np.mean(h_mid.astype(np.float64) ** 2) + 1e-6) * w
    assert rel_err(n, want) < 1e-6


def test_layer_tail_argument_errors(hip):
    from finchmoe_amd import FinchError
    with pytest.raises(FinchError) as e:
        hip.layer_tail_dev(12345, 16, 16, 16, 8, 16, 16, None, 1e-6, 16, None)
    assert e.value.status == fb.ERR_ARG


def _route(hip, logits, K, seg=None):
    import torch
    d_l = torch.from_numpy(np.ascontiguousarray(logits, np.float32)).cuda()
    d_idx = torch.full((K,), -7, dtype=torch.int32, device="cuda")
    d_w = torch.zeros(K, device="cuda")
    d_p = torch.full((10,), 9.0, device="cuda")
    d_seg = None if seg is None else torch.tensor([seg], dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    hip.route_topk_dev(d_l.data_ptr(), logits.size, K, None if seg is None else d_seg.data_ptr(),
                       d_idx.data_ptr(), d_w.data_ptr(), d_p.data_ptr())
    hip.sync()
    return d_idx.cpu().numpy(), d_w.cpu().numpy(), d_p.cpu().numpy()


@pytest.mark.parametrize("n,K", [(256, 8), (256, 1), (64, 8), (100, 5), (1000, 8), (8, 8)])
def test_route_matches_reference_scan(hip, orc, n, K):
    """Indices in the reference's slot order (exact), weights within rounding of the
    sequential softmax sum."""
    rng = np.random.default_rng(n * 10 + K)
    for trial in range(6):
        logits = (rng.standard_normal(n) * (1 + trial)).astype(np.float32)
        idx, w, p = _route(hip, logits, K, seg=0.25 * trial)
        ref_idx, ref_val = orc.topk(orc.softmax(logits), K)
        ref_w = orc.normalize_weights(ref_val)
        assert np.array_equal(idx, ref_idx), (trial, idx, ref_idx)
        assert np.abs(w - ref_w).max() <= 2e-6 * ref_w.max()
        assert np.array_equal(p[:K], w) and not p[K:8].any() and p[9] == 0
        assert p[8] == np.float32(0.25 * trial)
        assert abs(float(w.sum()) - 1) < 1e-6


def test_route_ties_and_order(hip, orc):
    """Equal scores: the earlier index is kept, and a later equal score does not replace it.
    Ascending scores: every element replaces the then-smallest slot."""
    logits = np.zeros(256, np.float32)
    idx, w, _ = _route(hip, logits, 8)
    assert np.array_equal(idx, np.arange(8))
    assert np.allclose(w, 1 / 8)
    logits = np.arange(256, dtype=np.float32) * 0.01
    idx, _, _ = _route(hip, logits, 8)
    assert np.array_equal(idx, orc.topk(orc.softmax(logits), 8)[0])
    assert sorted(idx.tolist()) == list(range(248, 256))
    logits = np.zeros(256, np.float32)
    logits[[5, 77, 200]] = 3.0
    logits[[6, 78]] = 3.0
    idx, _, _ = _route(hip, logits, 4)
    assert np.array_equal(idx, orc.topk(orc.softmax(logits), 4)[0])


def test_moe_half_of_a_layer_on_device(orc):
    """routing GEMV -> route -> routed experts -> layer tail without a host round trip
    (infer.m:9285-9760), against the same chain on the CPU oracle."""
    from finchmoe_amd import FinchHip
    hip = FinchHip(0)       # its own expert store
    try:
        _moe_half(hip, orc)
    finally:
        hip.close()


def _moe_half(hip, orc):
    import torch
    rng = np.random.default_rng(31)
    Hh, Ii, Ee, Kk = 2048, 512, 16, 8
    lo = F.expert_layout(Hh, Ii, 3)
    blob = F.synth_expert_layer(rng, Ee, Hh, Ii, 3)
    hip.experts_config(1, Ee, Hh, Ii, 64, 3, 0)
    hip.experts_upload_layer(0, blob)
    gate = F.synth_affine_tensor(rng, Ee, Hh, 8, "bf16")
    seg = F.synth_affine_tensor(rng, 1, Hh, 8, "bf16")
    sgt = F.synth_affine_tensor(rng, Ii, Hh, 4, "bf16")
    sut = F.synth_affine_tensor(rng, Ii, Hh, 4, "bf16")
    sdt = F.synth_affine_tensor(rng, Hh, Ii, 4, "bf16")
    t_gate = hip.tensor_register(*gate[1:], Ee, Hh, 8)
    t_seg = hip.tensor_register(*seg[1:], 1, Hh, 8)
    t_sg = hip.tensor_register(*sgt[1:], Ii, Hh, 4)
    t_su = hip.tensor_register(*sut[1:], Ii, Hh, 4)
    t_sd = hip.tensor_register(*sdt[1:], Hh, Ii, 4)
    x = rng.standard_normal(Hh).astype(np.float32)
    h_mid = rng.standard_normal(Hh).astype(np.float32)
    nw = _bf16(1.0 + 0.1 * rng.standard_normal(Hh))
    d_x, d_hmid = torch.from_numpy(x).cuda(), torch.from_numpy(h_mid).cuda()
    d_nw = torch.from_numpy(nw.view(np.int16)).cuda()
    d_log, d_seg = torch.empty(Ee, device="cuda"), torch.empty(1, device="cuda")
    d_sg, d_su = torch.empty(Ii, device="cuda"), torch.empty(Ii, device="cuda")
    d_idx = torch.empty(Kk, dtype=torch.int32, device="cuda")
    d_w, d_p = torch.empty(Kk, device="cuda"), torch.empty(10, device="cuda")
    d_moe, d_eo = torch.empty(Hh, device="cuda"), torch.empty(Kk, Hh, device="cuda")
    d_hid, d_next = torch.empty(Hh, device="cuda"), torch.empty(Hh, device="cuda")
    torch.cuda.synchronize()
    hip.matvec_batch_dev([t_gate, t_seg, t_sg, t_su], d_x.data_ptr(),
                         [d_log.data_ptr(), d_seg.data_ptr(), d_sg.data_ptr(), d_su.data_ptr()])
    hip.route_topk_dev(d_log.data_ptr(), Ee, Kk, d_seg.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(),
                       d_p.data_ptr())
    hip.moe_decode_dev(0, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), Kk, d_moe.data_ptr(),
                       d_eo.data_ptr())
    hip.layer_tail_dev(t_sd, d_hmid.data_ptr(), d_eo.data_ptr(), d_p.data_ptr(), Kk, d_sg.data_ptr(),
                       d_su.data_ptr(), d_nw.data_ptr(), 1e-6, d_hid.data_ptr(), d_next.data_ptr())
    hip.sync()
    # the same chain on the CPU
    logits = orc.dequant_matvec(*gate[1:], x, Ee, Hh, 8)
    segv = orc.dequant_matvec(*seg[1:], x, 1, Hh, 8)
    sg = orc.dequant_matvec(*sgt[1:], x, Ii, Hh, 4)
    su = orc.dequant_matvec(*sut[1:], x, Ii, Hh, 4)
    ridx, rval = orc.topk(orc.softmax(logits), Kk)
    rw = orc.normalize_weights(rval)
    assert np.array_equal(d_idx.cpu().numpy(), ridx)
    _, ref_eo = orc.moe_experts_forward(blob, x, ridx, rw, Hh, Ii, 3)
    params = np.zeros(10, np.float32)
    params[:Kk] = rw
    params[8] = segv[0]
    ref_h, ref_n = orc.layer_tail(*sdt[1:], h_mid, ref_eo, params, Kk, sg, su, nw)
    assert_parity(d_hid.cpu().numpy(), ref_h, "hidden")
    assert_parity(d_next.cpu().numpy(), ref_n, "next input")
    # the shorter chain: no buffer for the per-expert vectors, the tail takes the experts' sum
    # (K = 0 with a vector) — identical results
    d_moe2 = torch.empty(Hh, device="cuda")
    d_hid2, d_next2 = torch.empty(Hh, device="cuda"), torch.empty(Hh, device="cuda")
    torch.cuda.synchronize()
    hip.moe_decode_dev(0, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), Kk, d_moe2.data_ptr(), None)
    hip.layer_tail_dev(t_sd, d_hmid.data_ptr(), d_moe2.data_ptr(), d_p.data_ptr(), 0, d_sg.data_ptr(),
                       d_su.data_ptr(), d_nw.data_ptr(), 1e-6, d_hid2.data_ptr(), d_next2.data_ptr())
    hip.sync()
    assert torch.equal(d_moe2, d_moe) and torch.equal(d_hid2, d_hid) and torch.equal(d_next2, d_next)
    # and the first two launches as one (the GEMV batch's last workgroup routes): identical
    keep = [t.clone() for t in (d_log, d_seg, d_sg, d_su, d_idx, d_w, d_p)]
    for rep in range(3):       # the ticket word must come back to zero every time
        for t in (d_log, d_seg, d_sg, d_su, d_w, d_p):
            t.zero_()
        d_idx.zero_()
        torch.cuda.synchronize()
        hip.matvec_batch_route_dev([t_gate, t_seg, t_sg, t_su], d_x.data_ptr(),
                                   [d_log.data_ptr(), d_seg.data_ptr(), d_sg.data_ptr(), d_su.data_ptr()],
                                   Kk, d_seg.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), d_p.data_ptr())
        hip.sync()
        for got, want in zip((d_log, d_seg, d_sg, d_su, d_idx, d_w, d_p), keep):
            assert torch.equal(got, want), rep
    # the experts and the tail as ONE launch (the reference's CMD3 from the expert dispatches to
    # the next layer's norm): bit for bit the two launches above, several times in a row (the
    # activation sets alternate and the ticket word must come back to zero), also between other
    # decode calls, and in the last layer's form (no next input)
    for rep in range(4):
        d_hid3 = torch.full((Hh,), 3.0, device="cuda")
        d_next3 = torch.full((Hh,), 5.0, device="cuda")
        torch.cuda.synchronize()
        hip.moe_decode_tail_dev(0, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), Kk, t_sd, d_hmid.data_ptr(),
                                d_p.data_ptr(), d_sg.data_ptr(), d_su.data_ptr(), d_nw.data_ptr(), 1e-6,
                                d_hid3.data_ptr(), d_next3.data_ptr())
        hip.sync()
        assert torch.equal(d_hid3, d_hid), rep
        assert torch.equal(d_next3, d_next), rep
        if rep == 1:
            hip.moe_decode_dev(0, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), Kk, d_moe2.data_ptr(), None)
            hip.sync()
            assert torch.equal(d_moe2, d_moe)
    d_hid4 = torch.full((Hh,), 3.0, device="cuda")
    torch.cuda.synchronize()
    hip.moe_decode_tail_dev(0, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), Kk, t_sd, d_hmid.data_ptr(),
                            d_p.data_ptr(), d_sg.data_ptr(), d_su.data_ptr(), None, 1e-6, d_hid4.data_ptr(), None)
    hip.sync()
    assert torch.equal(d_hid4, d_hid)
    # the whole MoE half in two launches (routing batch; routing + experts + tail): every
    # intermediate and both results bit for bit the chain above, three times in a row
    for rep in range(3):
        o_log, o_seg = torch.zeros(Ee, device="cuda"), torch.zeros(1, device="cuda")
        o_sg, o_su = torch.zeros(Ii, device="cuda"), torch.zeros(Ii, device="cuda")
        o_idx = torch.zeros(Kk, dtype=torch.int32, device="cuda")
        o_w, o_p = torch.zeros(Kk, device="cuda"), torch.full((10,), 9.0, device="cuda")
        o_hid, o_next = torch.zeros(Hh, device="cuda"), torch.zeros(Hh, device="cuda")
        torch.cuda.synchronize()
        hip.moe_layer_dev(0, [t_gate, t_seg, t_sg, t_su], d_x.data_ptr(), Kk, t_sd, d_hmid.data_ptr(),
                          d_nw.data_ptr(), 1e-6, o_log.data_ptr(), o_seg.data_ptr(), o_sg.data_ptr(),
                          o_su.data_ptr(), o_idx.data_ptr(), o_w.data_ptr(), o_p.data_ptr(), o_hid.data_ptr(),
                          o_next.data_ptr())
        hip.sync()
        for got, want in zip((o_log, o_seg, o_sg, o_su, o_idx, o_w, o_p), keep):
            assert torch.equal(got, want), rep
        assert torch.equal(o_hid, d_hid) and torch.equal(o_next, d_next), rep
    # fewer slots than eight, and a slot with an index outside the store (weight 0 upstream)
    idx5 = d_idx.clone()
    idx5[2] = Ee + 7
    for kk, ix in ((5, d_idx), (Kk, idx5)):
        d_sum = torch.empty(Hh, device="cuda")
        d_ha, d_na = torch.empty(Hh, device="cuda"), torch.empty(Hh, device="cuda")
        d_hb, d_nb = torch.empty(Hh, device="cuda"), torch.empty(Hh, device="cuda")
        torch.cuda.synchronize()
        hip.moe_decode_dev(0, d_x.data_ptr(), ix.data_ptr(), d_w.data_ptr(), kk, d_sum.data_ptr(), None)
        hip.layer_tail_dev(t_sd, d_hmid.data_ptr(), d_sum.data_ptr(), d_p.data_ptr(), 0, d_sg.data_ptr(),
                           d_su.data_ptr(), d_nw.data_ptr(), 1e-6, d_ha.data_ptr(), d_na.data_ptr())
        hip.moe_decode_tail_dev(0, d_x.data_ptr(), ix.data_ptr(), d_w.data_ptr(), kk, t_sd, d_hmid.data_ptr(),
                                d_p.data_ptr(), d_sg.data_ptr(), d_su.data_ptr(), d_nw.data_ptr(), 1e-6,
                                d_hb.data_ptr(), d_nb.data_ptr())
        hip.sync()
        assert torch.equal(d_hb, d_ha) and torch.equal(d_nb, d_na), kk
    for t in (t_gate, t_seg, t_sg, t_su, t_sd):
        hip.tensor_release(t)
