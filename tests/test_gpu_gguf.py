"""GPU parity of the GGUF Q4_K / Q6_K expert path against the CPU oracle, through the C ABI.
Dequantized weights bit-exact; GEMV outputs within 1e-3 / cosine 0.99999."""
import numpy as np
import pytest

from finchmoe_amd import binding as fb
from finchmoe_amd import formats as F
from .conftest import assert_parity, rel_err

pytestmark = pytest.mark.gpu

H, I, E = 2048, 512, 10


@pytest.fixture(scope="module")
def gstore(hip):
    rng = np.random.default_rng(77)
    layers = [F.synth_gguf_layer(rng, E, H, I) for _ in range(3)]
    hip.gguf_config(3, E, H, I, (fb.Q4_K, fb.Q4_K, fb.Q6_K))
    for l, (g, u, d) in enumerate(layers):
        hip.gguf_upload_layer(l, g, u, d)
    return layers


def _slab(arr, e, rows, cols, gtype):
    n = rows * F.gguf_row_bytes(cols, gtype)
    return arr[e * n:(e + 1) * n]


def test_gguf_dequant_bit_exact(hip, orc, gstore):
    gate, up, down = gstore[1]
    for e in (0, 7):
        for which, arr, rows, cols, t in ((fb.GATE, gate, I, H, 12), (fb.UP, up, I, H, 12),
                                          (fb.DOWN, down, H, I, 14)):
            ref = orc.gguf_dequant(_slab(arr, e, rows, cols, t), rows, cols, t)
            got = hip.gguf_dequant_expert(1, e, which)
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (e, which)


def test_gguf_decode_matches_oracle(hip, orc, gstore):
    rng = np.random.default_rng(3)
    for layer in range(3):
        gate, up, down = gstore[layer]
        x = rng.standard_normal(H).astype(np.float32)
        idx, w = orc.route(rng.standard_normal(E).astype(np.float32), 8)
        ref, ref_eo = orc.moe_gguf_forward(gate, up, down, x, idx, w, H, I)
        out, eo = hip.gguf_moe_decode(layer, x, idx, w)
        assert_parity(eo, ref_eo, "expert_out layer %d" % layer)
        r, _ = assert_parity(out, ref, "layer %d" % layer)
        assert r < 5e-5, r
        again, _ = hip.gguf_moe_decode(layer, x, idx, w)
        assert np.array_equal(again, out)


def test_gguf_accumulate_guard_and_k(hip, orc, gstore):
    """moe_out is accumulated into (infer.m:3340); K < 8; guard with nothing to drop."""
    rng = np.random.default_rng(4)
    gate, up, down = gstore[0]
    x = rng.standard_normal(H).astype(np.float32)
    idx, w = orc.route(rng.standard_normal(E).astype(np.float32), 3)
    ref, _ = orc.moe_gguf_forward(gate, up, down, x, idx, w, H, I, guard=1)
    base = rng.standard_normal(H).astype(np.float32)
    out, _ = hip.gguf_moe_decode(0, x, idx, w, flags=fb.ACCUMULATE | fb.GUARD, out=base.copy())
    assert rel_err(out, base.astype(np.float64) + ref) < 1e-4


def test_gguf_step_and_small_chunk(hip, orc, gstore):
    import torch
    rng = np.random.default_rng(5)
    L, K = 3, 8
    x = rng.standard_normal((L, H)).astype(np.float32)
    idx = np.stack([orc.route(rng.standard_normal(E).astype(np.float32), K)[0] for _ in range(L)])
    w = np.stack([orc.normalize_weights(rng.random(K).astype(np.float32)) for _ in range(L)])
    dx, di, dw = (torch.from_numpy(a).cuda() for a in (x, idx, w))
    dout = torch.empty(L, H, device="cuda")
    torch.cuda.synchronize()
    hip.gguf_moe_decode_step_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K, dout.data_ptr())
    hip.sync()
    out = dout.cpu().numpy()
    for l in range(L):
        ref, _ = orc.moe_gguf_forward(*gstore[l], x[l], idx[l], w[l], H, I)
        assert_parity(out[l], ref, "layer %d" % l)
        single, _ = hip.gguf_moe_decode(l, x[l], idx[l], w[l])
        assert np.array_equal(single, out[l])
    # 8-position chunk on one layer == per-position calls
    chunk = hip.gguf_moe_prefill(2, np.repeat(x[:1], 8, 0) * np.arange(1, 9, dtype=np.float32)[:, None],
                                 np.tile(idx[0], (8, 1)), np.tile(w[0], (8, 1)))
    for m in range(8):
        single, _ = hip.gguf_moe_decode(2, x[0] * np.float32(m + 1), idx[0], w[0])
        assert np.array_equal(chunk[m], single)
    # 20 positions with their own routing (beyond 8 positions the per-position products are the three
    # streaming launches, up to 8 the one launch): still the per-position calls, bit for bit
    M = 20
    X = rng.standard_normal((M, H)).astype(np.float32)
    cidx = np.stack([orc.route(rng.standard_normal(E).astype(np.float32), K)[0] for _ in range(M)])
    cw = np.stack([orc.normalize_weights(rng.random(K).astype(np.float32)) for _ in range(M)])
    chunk = hip.gguf_moe_prefill(1, X, cidx, cw)
    for m in range(M):
        single, _ = hip.gguf_moe_decode(1, X[m], cidx[m], cw[m])
        assert np.array_equal(chunk[m], single), m


@pytest.mark.parametrize("gtype,out_dim,in_dim", [(12, 64, 2048), (14, 96, 512), (14, 7, 1024),
                                                  (12, 33, 256), (14, 16, 4096)])
def test_gguf_single_matvec(hip, orc, gtype, out_dim, in_dim):
    rng = np.random.default_rng(out_dim + in_dim)
    W = F.synth_gguf_tensor(rng, out_dim, in_dim, gtype)
    x = rng.standard_normal(in_dim).astype(np.float32)
    ref = orc.dequant_matvec(W, None, None, x, out_dim, in_dim, 10 if gtype == 12 else 11)
    got = hip.gguf_matvec(W, gtype, x, out_dim, in_dim)
    assert_parity(got, ref, "matvec")


def test_gguf_q4k_down_and_errors(orc):
    from finchmoe_amd import FinchHip, FinchError
    rng = np.random.default_rng(9)
    h, i, e = 1024, 256, 4
    gate, up, down = F.synth_gguf_layer(rng, e, h, i, (12, 12, 12))
    ctx = FinchHip(0)
    try:
        with pytest.raises(FinchError) as err:
            ctx.gguf_config(1, e, h, i, (fb.Q6_K, fb.Q4_K, fb.Q6_K))   # fused gate/up is Q4_K only
        assert err.value.status == fb.ERR_UNSUPPORTED
        ctx.gguf_config(1, e, h, i, (fb.Q4_K, fb.Q4_K, fb.Q4_K))
        x = rng.standard_normal(h).astype(np.float32)
        idx = np.array([3, 1], np.int32)
        w = np.array([0.4, 0.6], np.float32)
        with pytest.raises(FinchError) as err:
            ctx.gguf_moe_decode(0, x, idx, w)
        assert err.value.status == fb.ERR_STATE
        ctx.gguf_upload_layer(0, gate, up, down)
        ref, _ = orc.moe_gguf_forward(gate, up, down, x, idx, w, h, i, types=(12, 12, 12))
        out, _ = ctx.gguf_moe_decode(0, x, idx, w)
        assert_parity(out, ref, "Q4_K down")
    finally:
        ctx.close()


@pytest.mark.parametrize("h,i,down_t,layers,K", [(1024, 256, 14, 2, 8), (512, 1024, 14, 1, 4),
                                                 (2048, 2048, 12, 1, 2), (1024, 512, 12, 3, 8)])
def test_gguf_streaming_shapes(orc, h, i, down_t, layers, K):
    """Every lane count of the streaming kernels (4, 8, 16 lanes per row, both down formats), shares
    of the launch that cross pair and layer boundaries, and an expert index outside the store
    (contributes nothing: its slot of expert_out is zero)."""
    import torch
    from finchmoe_amd import FinchHip
    rng = np.random.default_rng(h + i + down_t)
    e = 10
    store = [F.synth_gguf_layer(rng, e, h, i, (12, 12, down_t)) for _ in range(layers)]
    ctx = FinchHip(0)
    try:
        ctx.gguf_config(layers, e, h, i, (fb.Q4_K, fb.Q4_K, down_t))
        for l, (g, u, d) in enumerate(store):
            ctx.gguf_upload_layer(l, g, u, d)
        x = rng.standard_normal((layers, h)).astype(np.float32)
        idx = np.stack([rng.permutation(e)[:K] for _ in range(layers)]).astype(np.int32)
        w = np.stack([orc.normalize_weights(rng.random(K).astype(np.float32)) for _ in range(layers)])
        idx[0, K - 1] = -1
        dx, di, dw = (torch.from_numpy(a).cuda() for a in (x, idx, w))
        dout = torch.empty(layers, h, device="cuda")
        deo = torch.empty(layers, K, h, device="cuda")
        torch.cuda.synchronize()
        ctx.gguf_moe_decode_step_dev(0, layers, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K,
                                     dout.data_ptr(), deo.data_ptr())
        ctx.sync()
        out, eo = dout.cpu().numpy(), deo.cpu().numpy()
        for l in range(layers):
            ok = idx[l] >= 0
            ref, ref_eo = orc.moe_gguf_forward(*store[l], x[l], np.where(ok, idx[l], 0).astype(np.int32),
                                               np.where(ok, w[l], 0).astype(np.float32), h, i,
                                               types=(12, 12, down_t))
            ref_eo[~ok] = 0
            assert_parity(eo[l], ref_eo, "expert_out layer %d" % l)
            assert_parity(out[l], ref, "layer %d" % l)
        assert not eo[0, K - 1].any()
    finally:
        ctx.close()


@pytest.mark.parametrize("h,i,down_t,layers,K", [(2048, 512, 14, 3, 8), (2048, 512, 14, 1, 5), (1024, 256, 14, 2, 8),
                                                 (1024, 512, 12, 3, 8)])
def test_gguf_one_launch_equals_three(orc, h, i, down_t, layers, K):
    """A caller that does not ask for the per-expert vectors gets the operator as one launch
    (gate/up, down by row blocks, slot-order sum in LDS).  Bit for bit the three launches (the same
    lane arithmetic and the same order of the sum), three calls in a row (the activation sets
    alternate and are re-marked), accumulation into out, an expert index outside the store; and
    within the bar of the oracle."""
    import torch
    from finchmoe_amd import FinchHip
    rng = np.random.default_rng(3 * h + i + down_t + K)
    e = 12
    store = [F.synth_gguf_layer(rng, e, h, i, (12, 12, down_t)) for _ in range(layers)]
    ctx = FinchHip(0)
    try:
        ctx.gguf_config(layers, e, h, i, (fb.Q4_K, fb.Q4_K, down_t))
        for l, (g, u, d) in enumerate(store):
            ctx.gguf_upload_layer(l, g, u, d)
        for rep in range(3):
            x = rng.standard_normal((layers, h)).astype(np.float32)
            idx = np.stack([rng.permutation(e)[:K] for _ in range(layers)]).astype(np.int32)
            w = np.stack([orc.normalize_weights(rng.random(K).astype(np.float32)) for _ in range(layers)])
            if rep == 1:
                idx[0, K - 1] = e + 3
            base = rng.standard_normal((layers, h)).astype(np.float32) if rep == 2 else np.zeros((layers, h), np.float32)
            flags = fb.ACCUMULATE if rep == 2 else 0
            dx, di, dw = (torch.from_numpy(a).cuda() for a in (x, idx, w))
            d_one, d_three = torch.from_numpy(base).cuda(), torch.from_numpy(base).cuda()
            torch.cuda.synchronize()
            try:
                ctx.set_kernel_forms(fb.FORM_GGUF_ONE_LAUNCH)
                ctx.gguf_moe_decode_step_dev(0, layers, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K,
                                             d_one.data_ptr(), None, flags)
                ctx.sync()
            finally:
                ctx.set_kernel_forms(0)
            try:
                ctx.set_kernel_forms(fb.FORM_GGUF_PHASES)
                ctx.gguf_moe_decode_step_dev(0, layers, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K,
                                             d_three.data_ptr(), None, flags)
                ctx.sync()
            finally:
                ctx.set_kernel_forms(0)
            one, three = d_one.cpu().numpy(), d_three.cpu().numpy()
            assert np.array_equal(one.view(np.uint32), three.view(np.uint32)), rep
            for l in range(layers):
                ok = (idx[l] >= 0) & (idx[l] < e)
                ref, _ = orc.moe_gguf_forward(*store[l], x[l], np.where(ok, idx[l], 0).astype(np.int32),
                                              np.where(ok, w[l], 0).astype(np.float32), h, i, types=(12, 12, down_t))
                assert_parity(one[l], base[l].astype(np.float64) + ref, "layer %d call %d" % (l, rep))
    finally:
        ctx.close()


@pytest.mark.parametrize("M,K,h,i,seed", [(40, 8, 2048, 512, 1), (97, 4, 1024, 256, 2), (32, 8, 512, 512, 3),
                                          (36, 4, 4096, 256, 4)])
def test_gguf_chunk_grouped_products(orc, M, K, h, i, seed):
    """Chunks of 32 positions and more on a Q4_K / Q4_K / Q6_K store take the grouped products
    (an expert streamed once per group of its positions, prefill_chunk_cmd3_batch_general's
    result, finchmoe/infer.m:10958-11059): every position equals its per-position call and the
    oracle within the bar; skewed routing gives items of every size, an expert index outside the
    store contributes nothing, the accumulate flag adds, and a repeat is bit-identical."""
    from finchmoe_amd import FinchHip
    rng = np.random.default_rng(seed)
    Ee = 12
    gate, up, down = F.synth_gguf_layer(rng, Ee, h, i)
    ctx = FinchHip(0)
    try:
        ctx.gguf_config(1, Ee, h, i, (fb.Q4_K, fb.Q4_K, fb.Q6_K))
        ctx.gguf_upload_layer(0, gate, up, down)
        X = rng.standard_normal((M, h)).astype(np.float32)
        # skewed: expert 0 in every position's set, the others random without repeats
        idx = np.stack([np.concatenate([[0], 1 + rng.permutation(Ee - 1)[:K - 1]]) for _ in range(M)]).astype(np.int32)
        w = rng.random((M, K)).astype(np.float32)
        idx[5, K - 1] = Ee + 3                                 # outside the store
        out = ctx.gguf_moe_prefill(0, X, idx, w)
        assert np.isfinite(out).all()
        assert np.array_equal(ctx.gguf_moe_prefill(0, X, idx, w), out)
        for m in range(M):
            keep = idx[m] < Ee
            single, _ = ctx.gguf_moe_decode(0, X[m], idx[m][keep], w[m][keep])
            assert rel_err(out[m], single) < 1e-3, (m, rel_err(out[m], single))
        for m in (0, 5, M - 1):
            keep = idx[m] < Ee
            ref, _ = orc.moe_gguf_forward(gate, up, down, X[m], idx[m][keep], w[m][keep], h, i)
            assert_parity(out[m], ref, "position %d" % m)
        base = rng.standard_normal((M, h)).astype(np.float32)
        acc = ctx.gguf_moe_prefill(0, X, idx, w, flags=fb.ACCUMULATE, out=base.copy())
        assert rel_err(acc, base + out) < 1e-6
    finally:
        ctx.close()


@pytest.mark.parametrize("gtype,out_dim,in_dim", [(12, 4096, 2048), (14, 4096, 1024), (14, 1024, 2048),
                                                  (12, 515, 512), (14, 100, 256), (12, 64, 4096)])
def test_gguf_dense_tensor_resident_matvec_and_embedding(hip, orc, gtype, out_dim, in_dim):
    """A Q4_K / Q6_K tensor registered with the reference's bits 10 / 11: fp32 values and the
    embedding rows bit for bit the oracle's gguf_dequant_row, the matvec within the bar (the
    streaming kernel where the shape allows it, the rows-per-wave kernel otherwise), also for
    several positions."""
    rng = np.random.default_rng(3 * out_dim + in_dim + gtype)
    W = F.synth_gguf_tensor(rng, out_dim, in_dim, gtype)
    bits = 10 if gtype == 12 else 11
    t = hip.tensor_register(W, None, None, out_dim, in_dim, bits=bits)
    try:
        ref_w = orc.gguf_dequant(W, out_dim, in_dim, gtype)
        if out_dim * in_dim <= 1 << 22:
            w32 = np.empty((out_dim, in_dim), np.float32)
            hip._chk(hip.L.fm_dequant_tensor(hip.h, t, None, w32.ctypes.data, None))
            assert np.array_equal(w32.view(np.uint32), ref_w.view(np.uint32))
        for tok in (0, out_dim - 1, out_dim // 3):
            row = hip.embed_lookup(t, tok, in_dim)
            assert np.array_equal(row.view(np.uint32), ref_w[tok].view(np.uint32))
        assert not hip.embed_lookup(t, out_dim, in_dim).any()          # outside the tensor: zeros
        x = rng.standard_normal(in_dim).astype(np.float32)
        ref = orc.dequant_matvec(W, None, None, x, out_dim, in_dim, bits)
        (got,) = hip.matvec_batch([t], x, [out_dim])
        assert_parity(got, ref, "resident GGUF matvec")
        X = rng.standard_normal((3, in_dim)).astype(np.float32)
        outs = hip.matvec_prefill(t, X, out_dim)
        for m in range(3):
            assert_parity(outs[m], orc.dequant_matvec(W, None, None, X[m], out_dim, in_dim, bits), "position %d" % m)
    finally:
        hip.tensor_release(t)


@pytest.mark.parametrize("gtype", [12, 14])
def test_gguf_vocabulary_projection_full_size(orc, gtype):
    """The vocabulary projection of a GGUF model at its real size, 248320 x 2048 (Q4_K: the
    streaming kernel; Q6_K: the rows-per-wave kernel): a few thousand sampled rows against the
    oracle, every output finite, and rows sampled from the embedding lookup bit for bit."""
    import torch
    from finchmoe_amd import FinchHip
    V, D = 248320, 2048
    rb = F.gguf_row_bytes(D, gtype)
    bsz = 144 if gtype == 12 else 210
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(17 + gtype)
    Wd = torch.empty(V * (D // 256), bsz, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
    n_d, d_off = (2, 0) if gtype == 12 else (1, 208)
    d = (torch.randn(V * (D // 256), n_d, device=dev, generator=gen).abs_() * 0.002).to(torch.float16)
    Wd[:, d_off:d_off + 2 * n_d] = d.view(torch.uint8)
    x = torch.randn(D, device=dev, generator=gen)
    out = torch.empty(V, device=dev)
    torch.cuda.synchronize()
    ctx = FinchHip(0)
    try:
        t = ctx.tensor_adopt(Wd.data_ptr(), None, None, V, D, bits=10 if gtype == 12 else 11)
        ctx.matvec_batch_dev([t], x.data_ptr(), [out.data_ptr()])
        ctx.sync()
        got = out.cpu().numpy()
        assert np.isfinite(got).all()
        rng = np.random.default_rng(5)
        rows = np.unique(np.concatenate([rng.integers(0, V, 3000), [0, 1, 2, 3, V - 4, V - 3, V - 2, V - 1]]))
        Wh = Wd.view(V, rb)[torch.from_numpy(rows).to(dev)].cpu().numpy()
        xh = x.cpu().numpy()
        ref = orc.dequant_matvec(Wh.reshape(-1), None, None, xh, len(rows), D, 10 if gtype == 12 else 11)
        assert_parity(got[rows], ref, "sampled rows of the vocabulary projection")
        ids = torch.tensor([0, 777, V - 1], dtype=torch.int32, device=dev)
        emb = torch.empty(3, D, device=dev)
        ctx.embed_lookup_dev(t, ids.data_ptr(), 3, emb.data_ptr())
        ctx.sync()
        for i, tok in enumerate((0, 777, V - 1)):
            rowb = Wd.view(V, rb)[tok].cpu().numpy()
            assert np.array_equal(emb[i].cpu().numpy().view(np.uint32),
                                  orc.gguf_dequant(rowb, 1, D, gtype)[0].view(np.uint32))
    finally:
        ctx.close()
