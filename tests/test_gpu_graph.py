"""A captured launch of the fused decode step replayed from a HIP graph: the dependency
counters of the kernel are cleared by the launch itself, so every replay must equal the eager
result for the inputs that are in the buffers at that time."""
import ctypes as C

import numpy as np
import pytest

from finchmoe_amd import binding as fb
from finchmoe_amd import formats as F

pytestmark = pytest.mark.gpu

H, I, E, K, L = 2048, 512, 16, 8, 6


def _hip():
    lib = C.CDLL("libamdhip64.so")
    for name, args in (("hipStreamBeginCapture", [C.c_void_p, C.c_int]),
                       ("hipStreamEndCapture", [C.c_void_p, C.POINTER(C.c_void_p)]),
                       ("hipGraphInstantiate", [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p,
                                                C.c_size_t]),
                       ("hipGraphLaunch", [C.c_void_p, C.c_void_p]),
                       ("hipGraphExecDestroy", [C.c_void_p]),
                       ("hipGraphDestroy", [C.c_void_p])):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = args
    return lib


def test_decode_step_replayed_from_graph():
    import torch
    from finchmoe_amd import FinchHip
    hip = _hip()
    rng = np.random.default_rng(31)
    ctx = FinchHip(0)
    try:
        ctx.experts_config(L, E, H, I, 64, 3, fb.SCALE_BF16)
        for l in range(L):
            ctx.experts_upload_layer(l, F.synth_expert_layer(rng, E, H, I, 3))
        d_x = torch.zeros(L, H, device="cuda")
        d_idx = torch.zeros(L, K, dtype=torch.int32, device="cuda")
        d_w = torch.zeros(L, K, device="cuda")
        d_out = torch.zeros(L, H, device="cuda")
        d_ref = torch.zeros(L, H, device="cuda")

        def new_inputs():
            d_x.copy_(torch.from_numpy(rng.standard_normal((L, H)).astype(np.float32)))
            idx = np.stack([rng.permutation(E)[:K] for _ in range(L)]).astype(np.int32)
            w = rng.random((L, K)).astype(np.float32)
            d_idx.copy_(torch.from_numpy(idx))
            d_w.copy_(torch.from_numpy(w / w.sum(1, keepdims=True)))
            torch.cuda.synchronize()

        def eager(dst):
            ctx.moe_decode_step_dev(0, L, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K, dst.data_ptr())
            ctx.sync()

        new_inputs()
        eager(d_ref)                       # scratch buffers and kernel attributes exist from here on
        stream = C.c_void_p(ctx.stream())
        graph, gexec = C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(stream, 2) == 0          # relaxed mode
        ctx.moe_decode_step_dev(0, L, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K, d_out.data_ptr())
        assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        for rep in range(4):
            if rep:
                new_inputs()
            eager(d_ref)                   # eager work of the same kind between the replays
            d_out.zero_()
            torch.cuda.synchronize()
            assert hip.hipGraphLaunch(gexec, stream) == 0
            ctx.sync()
            assert np.array_equal(d_out.cpu().numpy(), d_ref.cpu().numpy()), rep
        # two replays in a row without anything in between
        assert hip.hipGraphLaunch(gexec, stream) == 0
        assert hip.hipGraphLaunch(gexec, stream) == 0
        ctx.sync()
        assert np.array_equal(d_out.cpu().numpy(), d_ref.cpu().numpy())
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
    finally:
        ctx.close()


def test_moe_half_of_a_layer_replayed_from_graph():
    """routing GEMVs -> route -> routed experts -> layer tail (four kinds of launch, two of them
    with counters or tickets in device memory) captured once and replayed with new inputs."""
    import torch
    from finchmoe_amd import FinchHip
    hip = _hip()
    rng = np.random.default_rng(32)
    Ee = 16
    ctx = FinchHip(0)
    try:
        ctx.experts_config(1, Ee, H, I, 64, 3, fb.SCALE_BF16)
        ctx.experts_upload_layer(0, F.synth_expert_layer(rng, Ee, H, I, 3))
        tens = [F.synth_affine_tensor(rng, r, c, b, "bf16")
                for (r, c, b) in ((Ee, H, 8), (1, H, 8), (I, H, 4), (I, H, 4), (H, I, 4))]
        t_gate, t_seg, t_sg, t_su, t_sd = [ctx.tensor_register(*t[1:], r, c, b) for t, (r, c, b) in
                                           zip(tens, ((Ee, H, 8), (1, H, 8), (I, H, 4), (I, H, 4), (H, I, 4)))]
        nw = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
        d_nw = torch.from_numpy((nw.view(np.uint32) >> 16).astype(np.uint16).view(np.int16)).cuda()
        d_x, d_hmid = torch.zeros(H, device="cuda"), torch.zeros(H, device="cuda")
        d_log, d_seg = torch.empty(Ee, device="cuda"), torch.empty(1, device="cuda")
        d_sg, d_su = torch.empty(I, device="cuda"), torch.empty(I, device="cuda")
        d_idx = torch.empty(K, dtype=torch.int32, device="cuda")
        d_w, d_p = torch.empty(K, device="cuda"), torch.empty(10, device="cuda")
        d_moe, d_eo = torch.empty(H, device="cuda"), torch.empty(K, H, device="cuda")
        outs = [torch.zeros(H, device="cuda") for _ in range(4)]     # hidden, next: graph / eager

        def chain(d_hid, d_next):
            ctx.matvec_batch_dev([t_gate, t_seg, t_sg, t_su], d_x.data_ptr(),
                                 [d_log.data_ptr(), d_seg.data_ptr(), d_sg.data_ptr(), d_su.data_ptr()])
            ctx.route_topk_dev(d_log.data_ptr(), Ee, K, d_seg.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(),
                               d_p.data_ptr())
            ctx.moe_decode_dev(0, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K, d_moe.data_ptr(),
                               d_eo.data_ptr())
            ctx.layer_tail_dev(t_sd, d_hmid.data_ptr(), d_eo.data_ptr(), d_p.data_ptr(), K, d_sg.data_ptr(),
                               d_su.data_ptr(), d_nw.data_ptr(), 1e-6, d_hid.data_ptr(), d_next.data_ptr())

        def new_inputs():
            d_x.copy_(torch.from_numpy(rng.standard_normal(H).astype(np.float32)))
            d_hmid.copy_(torch.from_numpy(rng.standard_normal(H).astype(np.float32)))
            torch.cuda.synchronize()

        new_inputs()
        chain(outs[2], outs[3])
        ctx.sync()
        stream = C.c_void_p(ctx.stream())
        graph, gexec = C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(stream, 2) == 0
        chain(outs[0], outs[1])
        assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        for rep in range(4):
            new_inputs()
            chain(outs[2], outs[3])
            ctx.sync()
            assert hip.hipGraphLaunch(gexec, stream) == 0
            ctx.sync()
            assert np.array_equal(outs[0].cpu().numpy(), outs[2].cpu().numpy()), rep
            assert np.array_equal(outs[1].cpu().numpy(), outs[3].cpu().numpy()), rep
            assert np.isfinite(outs[1].cpu().numpy()).all() and np.abs(outs[1].cpu().numpy()).max() > 0
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
    finally:
        ctx.close()


def test_scratch_is_pinned_by_a_capture_and_reserved_beforehand():
    """A graph holds the scratch addresses of its capture: sizes are reserved first
    (fm_reserve), a later call that would have to grow the scratch is refused with a state
    error instead of moving it, the graph still replays correctly, and fm_release_graphs lifts
    the pin."""
    import torch
    from finchmoe_amd import FinchHip, FinchError
    hip = _hip()
    rng = np.random.default_rng(41)
    ctx = FinchHip(0)
    try:
        ctx.experts_config(L, E, H, I, 64, 3, fb.SCALE_BF16)
        for l in range(L):
            ctx.experts_upload_layer(l, F.synth_expert_layer(rng, E, H, I, 3))
        x = torch.from_numpy(rng.standard_normal((L, H)).astype(np.float32)).cuda()
        idx = torch.from_numpy(np.stack([rng.permutation(E)[:K] for _ in range(L)]).astype(np.int32)).cuda()
        w = torch.full((L, K), 1.0 / K, device="cuda")
        d_out, d_ref = torch.zeros(L, H, device="cuda"), torch.zeros(L, H, device="cuda")
        ctx.reserve(n_groups=2)                       # enough for steps of two layers
        ctx.moe_decode_step_dev(0, 2, x.data_ptr(), idx.data_ptr(), w.data_ptr(), K, d_ref.data_ptr())
        ctx.sync()
        stream = C.c_void_p(ctx.stream())
        graph, gexec = C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(stream, 2) == 0
        ctx.moe_decode_step_dev(0, 2, x.data_ptr(), idx.data_ptr(), w.data_ptr(), K, d_out.data_ptr())
        assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        with pytest.raises(FinchError) as e:          # six layers need more scratch than reserved
            ctx.moe_decode_step_dev(0, L, x.data_ptr(), idx.data_ptr(), w.data_ptr(), K, d_ref.data_ptr())
        assert e.value.status == fb.ERR_STATE and "fm_reserve" in str(e.value)
        assert hip.hipGraphLaunch(gexec, stream) == 0
        ctx.sync()
        assert torch.equal(d_out[:2], d_ref[:2])
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
        ctx.release_graphs()
        ctx.moe_decode_step_dev(0, L, x.data_ptr(), idx.data_ptr(), w.data_ptr(), K, d_out.data_ptr())
        ctx.sync()
        assert torch.isfinite(d_out).all() and torch.equal(d_out[:2], d_ref[:2])
    finally:
        ctx.close()
