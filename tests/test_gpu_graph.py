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
