"""The C host layer (libfinchops.so) that carries the reference's operator names
(fast_dequant_matvec, BatchMatvecSpec + fast_batch_matvec, moe_experts_forward,
gpu_gguf_experts_forward, cpu_softmax/topk/normalize).  Routing helpers are checked on the
CPU; the compute entry points on the GPU against the oracle."""
import ctypes as C
import os

import numpy as np
import pytest

from finchmoe_amd import formats as F
from .conftest import assert_parity, rel_err

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class BatchMatvecSpec(C.Structure):   # finchmoe/infer.m:3401-3411
    _fields_ = [("W", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p),
                ("out_cpu", C.c_void_p), ("out_dim", C.c_uint32), ("in_dim", C.c_uint32),
                ("group_size", C.c_uint32), ("batch_slot", C.c_int), ("bits", C.c_int)]


@pytest.fixture(scope="module")
def ops():
    from finchmoe_amd import binding
    binding.load()      # shares the HIP runtime (see binding.load)
    L = C.CDLL(os.path.join(ROOT, "finchmoe_amd", "libfinchops.so"))
    vp, i = C.c_void_p, C.c_int
    L.fast_dequant_matvec.argtypes = [vp, vp, vp, vp, vp, i, i, i, i]
    L.fast_batch_matvec.argtypes = [vp, C.c_uint32, C.POINTER(BatchMatvecSpec), i]
    L.fast_prefill_matvec.argtypes = [vp, vp, vp, vp, vp, i, i, i, i, i]
    L.finch_ops_load_expert_layer.argtypes = [i, vp, C.c_size_t]
    L.finch_ops_load_gguf_layer.argtypes = [i, vp, C.c_size_t, vp, C.c_size_t, vp, C.c_size_t]
    L.moe_experts_forward.argtypes = [i, vp, vp, vp, i, vp]
    L.gpu_gguf_experts_forward.argtypes = [i, vp, vp, vp, i, vp]
    L.moe_experts_forward_chunk.argtypes = [i, vp, vp, vp, i, i, vp]
    L.cpu_softmax.argtypes = [vp, i]
    L.cpu_topk.argtypes = [vp, i, i, vp, vp]
    L.cpu_normalize_weights.argtypes = [vp, i]
    L.finch_ops_last_error.restype = C.c_char_p
    return L


def test_routing_helpers_match_oracle(ops, orc):
    rng = np.random.default_rng(0)
    for n, K in ((256, 8), (16, 4), (8, 8)):
        logits = rng.standard_normal(n).astype(np.float32)
        p = logits.copy()
        ops.cpu_softmax(p.ctypes.data, n)
        assert np.array_equal(p, orc.softmax(logits))
        idx = np.empty(K, np.int32)
        val = np.empty(K, np.float32)
        ops.cpu_topk(p.ctypes.data, n, K, idx.ctypes.data, val.ctypes.data)
        ridx, rval = orc.topk(p, K)
        assert np.array_equal(idx, ridx) and np.array_equal(val, rval)
        ops.cpu_normalize_weights(val.ctypes.data, K)
        assert np.array_equal(val, orc.normalize_weights(rval))
    ties = np.array([0.25, 0.5, 0.25, 0.5, 0.25], np.float32)
    idx = np.empty(2, np.int32)
    val = np.empty(2, np.float32)
    ops.cpu_topk(ties.ctypes.data, 5, 2, idx.ctypes.data, val.ctypes.data)
    assert idx.tolist() == orc.topk(ties, 2)[0].tolist()


def test_calls_before_init_fail_without_computing(ops):
    x = np.ones(2048, np.float32)
    out = np.full(64, 7.0, np.float32)
    ops.finch_ops_shutdown()
    ops.fast_dequant_matvec(x.ctypes.data, x.ctypes.data, x.ctypes.data, x.ctypes.data,
                            out.ctypes.data, 64, 2048, 64, 4)
    assert ops.finch_ops_last_status() != 0 and np.all(out == 7.0)


@pytest.mark.gpu
def test_host_ops_on_gpu(ops, orc):
    H, I, E = 2048, 512, 6
    rng = np.random.default_rng(11)
    assert ops.finch_ops_init(0) == 0, ops.finch_ops_last_error()
    try:
        # BatchMatvecSpec: qkv + z from one x (infer.m:8119-8122)
        _, Wq, Sq, Bq = F.synth_affine_tensor(rng, 1024, H, 4)
        _, Wz, Sz, Bz = F.synth_affine_tensor(rng, 512, H, 4)
        x = rng.standard_normal(H).astype(np.float32)
        oq, oz = np.empty(1024, np.float32), np.empty(512, np.float32)
        specs = (BatchMatvecSpec * 2)(
            BatchMatvecSpec(Wq.ctypes.data, Sq.ctypes.data, Bq.ctypes.data, oq.ctypes.data, 1024, H, 64, 0, 4),
            BatchMatvecSpec(Wz.ctypes.data, Sz.ctypes.data, Bz.ctypes.data, oz.ctypes.data, 512, H, 64, 1, 4))
        ops.fast_batch_matvec(x.ctypes.data, H, specs, 2)
        assert ops.finch_ops_last_status() == 0, ops.finch_ops_last_error()
        assert_parity(oq, orc.dequant_matvec(Wq, Sq, Bq, x, 1024, H, 4), "qkv")
        assert_parity(oz, orc.dequant_matvec(Wz, Sz, Bz, x, 512, H, 4), "z")
        # single matvec, second call hits the resident copy
        o1 = np.empty(512, np.float32)
        for _ in range(2):
            ops.fast_dequant_matvec(Wz.ctypes.data, Sz.ctypes.data, Bz.ctypes.data, x.ctypes.data,
                                    o1.ctypes.data, 512, H, 64, 4)
        assert np.array_equal(o1, oz)
        # GGUF tensor through the same call (bits 10 / 11, scales NULL)
        Wg = F.synth_gguf_tensor(rng, 96, 512, 14)
        xg = rng.standard_normal(512).astype(np.float32)
        og = np.empty(96, np.float32)
        ops.fast_dequant_matvec(Wg.ctypes.data, None, None, xg.ctypes.data, og.ctypes.data, 96, 512, 64, 11)
        assert_parity(og, orc.dequant_matvec(Wg, None, None, xg, 96, 512, 11), "Q6_K")
        # M positions
        X = rng.standard_normal((4, H)).astype(np.float32)
        om = np.empty((4, 512), np.float32)
        ops.fast_prefill_matvec(Wz.ctypes.data, Sz.ctypes.data, Bz.ctypes.data, X.ctypes.data,
                                om.ctypes.data, 512, H, 64, 4, 4)
        for m in range(4):
            assert_parity(om[m], orc.dequant_matvec(Wz, Sz, Bz, X[m], 512, H, 4), "pos %d" % m)
        # routed experts: += into moe_out, CPU-path guard semantics
        blob = F.synth_expert_layer(rng, E, H, I, 3)
        assert ops.finch_ops_config_experts(2, E, H, I, 3) == 0
        assert ops.finch_ops_load_expert_layer(1, blob.ctypes.data, blob.size) == 0
        idx, w = orc.route(rng.standard_normal(E).astype(np.float32), 4)
        base = rng.standard_normal(H).astype(np.float32)
        moe = base.copy()
        assert ops.moe_experts_forward(1, x.ctypes.data, idx.ctypes.data, w.ctypes.data, 4, moe.ctypes.data) == 1
        ref, _ = orc.moe_experts_forward(blob, x, idx, w, H, I, 3, guard=1)
        assert rel_err(moe, base.astype(np.float64) + ref) < 1e-5
        # layer 0 was never loaded: returns 0 ("fall back"), leaves moe_out alone
        keep = moe.copy()
        assert ops.moe_experts_forward(0, x.ctypes.data, idx.ctypes.data, w.ctypes.data, 4, moe.ctypes.data) == 0
        assert np.array_equal(moe, keep)
        # chunk of positions
        Xc = rng.standard_normal((3, H)).astype(np.float32)
        ic = np.tile(idx, (3, 1)).astype(np.int32)
        wc = np.tile(w, (3, 1)).astype(np.float32)
        oc = np.zeros((3, H), np.float32)
        assert ops.moe_experts_forward_chunk(1, Xc.ctypes.data, ic.ctypes.data, wc.ctypes.data, 3, 4, oc.ctypes.data) == 1
        for m in range(3):
            r, _ = orc.moe_experts_forward(blob, Xc[m], idx, w, H, I, 3)
            assert_parity(oc[m], r, "chunk pos %d" % m)
        # GGUF experts
        g, u, d = F.synth_gguf_layer(rng, E, H, I)
        assert ops.finch_ops_config_gguf_experts(1, E, H, I, 12, 12, 14) == 0
        assert ops.finch_ops_load_gguf_layer(0, g.ctypes.data, g.size, u.ctypes.data, u.size, d.ctypes.data, d.size) == 0
        moe = np.zeros(H, np.float32)
        assert ops.gpu_gguf_experts_forward(0, x.ctypes.data, idx.ctypes.data, w.ctypes.data, 4, moe.ctypes.data) == 1
        refg, _ = orc.moe_gguf_forward(g, u, d, x, idx, w, H, I, guard=1)
        assert_parity(moe, refg, "gguf experts")
    finally:
        ops.finch_ops_shutdown()


@pytest.mark.gpu
def test_reference_gdn_batch_with_raw_bf16_specs(ops, orc):
    """The reference's own decode batch {qkv 8192, z 4096, b 32, a 32} (infer.m:8118-8122):
    qkv and z are 4-bit, in_proj_b / in_proj_a stay BF16 in the reference's checkpoints
    (quantize_non_experts.py:103-107) and arrive with scales == biases == NULL.  Also the
    routing gate [256, 2048] and the shared expert's gate [1, 2048] as single BF16 matvecs
    (cpu_dequant_matvec's raw branch, infer.m:1689-1701)."""
    H = 2048
    rng = np.random.default_rng(21)
    assert ops.finch_ops_init(0) == 0, ops.finch_ops_last_error()
    try:
        _, Wq, Sq, Bq = F.synth_affine_tensor(rng, 8192, H, 4)
        _, Wz, Sz, Bz = F.synth_affine_tensor(rng, 4096, H, 4)
        Wb = F.bf16_trunc(rng.standard_normal((32, H)).astype(np.float32) * np.float32(0.05))
        Wa = F.bf16_trunc(rng.standard_normal((32, H)).astype(np.float32) * np.float32(0.05))
        x = rng.standard_normal(H).astype(np.float32)
        oq, oz = np.full(8192, np.nan, np.float32), np.full(4096, np.nan, np.float32)
        ob, oa = np.full(32, np.nan, np.float32), np.full(32, np.nan, np.float32)
        specs = (BatchMatvecSpec * 4)(
            BatchMatvecSpec(Wq.ctypes.data, Sq.ctypes.data, Bq.ctypes.data, oq.ctypes.data, 8192, H, 64, 0, 4),
            BatchMatvecSpec(Wz.ctypes.data, Sz.ctypes.data, Bz.ctypes.data, oz.ctypes.data, 4096, H, 64, 1, 0),
            BatchMatvecSpec(Wb.ctypes.data, None, None, ob.ctypes.data, 32, H, 64, 2, 0),
            BatchMatvecSpec(Wa.ctypes.data, None, None, oa.ctypes.data, 32, H, 64, 3, 4))
        ops.fast_batch_matvec(x.ctypes.data, H, specs, 4)
        assert ops.finch_ops_last_status() == 0, ops.finch_ops_last_error()
        assert_parity(oq, orc.dequant_matvec(Wq, Sq, Bq, x, 8192, H, 4), "qkv")
        assert_parity(oz, orc.dequant_matvec(Wz, Sz, Bz, x, 4096, H, 4), "z (bits 0 = 4)")
        assert_parity(ob, orc.dequant_matvec(Wb, None, None, x, 32, H, 0), "in_proj_b (BF16)")
        assert_parity(oa, orc.dequant_matvec(Wa, None, None, x, 32, H, 0), "in_proj_a (BF16)")
        # single BF16 matvecs: routing gate and shared-expert gate score
        Wg = F.bf16_trunc(rng.standard_normal((256, H)).astype(np.float32) * np.float32(0.05))
        og = np.empty(256, np.float32)
        for _ in range(2):    # second call hits the resident copy
            ops.fast_dequant_matvec(Wg.ctypes.data, None, None, x.ctypes.data, og.ctypes.data, 256, H, 64, 0)
            assert ops.finch_ops_last_status() == 0, ops.finch_ops_last_error()
        assert_parity(og, orc.dequant_matvec(Wg, None, None, x, 256, H, 0), "mlp.gate (BF16)")
        Ws = F.bf16_trunc(rng.standard_normal((1, H)).astype(np.float32))
        os_ = np.empty(1, np.float32)
        ops.fast_dequant_matvec(Ws.ctypes.data, None, None, x.ctypes.data, os_.ctypes.data, 1, H, 64, 0)
        ref = orc.dequant_matvec(Ws, None, None, x, 1, H, 0)
        assert abs(float(os_[0]) - float(ref[0])) <= 1e-3 * max(1.0, abs(float(ref[0])))
        # a failing batch never leaves its outputs uninitialised (the call returns void)
        bad = (BatchMatvecSpec * 1)(
            BatchMatvecSpec(Wq.ctypes.data, Sq.ctypes.data, Bq.ctypes.data, oq.ctypes.data, 8192, H, 64, 0, 5))
        oq[:] = np.nan
        ops.fast_batch_matvec(x.ctypes.data, H, bad, 1)
        assert ops.finch_ops_last_status() != 0 and np.all(oq == 0.0)
    finally:
        ops.finch_ops_shutdown()
