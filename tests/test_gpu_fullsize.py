"""The benchmark's full sizes (40 layers x 256 experts of 3-bit g64 weights resident, 14.09 GB;
512-position chunk on 256 experts), checked through properties that do not need the oracle to
process 14 GB: the 40-layer step equals the 40 single-layer calls bit for bit; the weighted sum
equals the per-expert outputs combined in slot order; sampled (layer, slot) expert outputs equal
the CPU oracle on the routed experts' bytes copied back; a prefill chunk equals the per-position
path.  Weights are generated on the device exactly as bench.py does."""
import numpy as np
import pytest

from finchmoe_amd import formats as F
from .conftest import assert_parity, cosine, rel_err

pytestmark = pytest.mark.gpu

H, I, E, K, L = 2048, 512, 256, 8, 40


@pytest.fixture(scope="module")
def full_store():
    import torch
    from bench import fill_affine_layer, zipf_routing
    from finchmoe_amd import FinchHip
    dev = torch.device("cuda:0")
    lo = F.expert_layout(H, I, 3)
    es = lo["expert_size"]
    gen = torch.Generator(device=dev)
    gen.manual_seed(2024)
    blob = torch.empty(L, E, es, dtype=torch.uint8, device=dev)
    for l in range(L):
        fill_affine_layer(blob[l], lo, 3, gen)
    torch.cuda.synchronize()       # the context's stream does not wait for torch's
    ctx = FinchHip(0)
    ctx.experts_config(L, E, H, I, 64, 3, 0)
    for l in range(L):
        ctx.experts_adopt_layer(l, blob[l].data_ptr(), E * es)
    idx, w = zipf_routing(np.random.default_rng(5), 2, L, E, K)
    yield ctx, blob, lo, idx, w
    ctx.close()
    del blob
    torch.cuda.empty_cache()


def test_full_step_equals_layer_calls_and_oracle(full_store, orc):
    import torch
    ctx, blob, lo, idx, w = full_store
    es = lo["expert_size"]
    rng = np.random.default_rng(6)
    x = rng.standard_normal((L, H)).astype(np.float32)
    d_x = torch.from_numpy(x).cuda()
    for tok in range(2):
        d_idx, d_w = torch.from_numpy(idx[tok]).cuda(), torch.from_numpy(w[tok]).cuda()
        d_out = torch.zeros(L, H, device="cuda")
        d_eo = torch.zeros(L, K, H, device="cuda")
        torch.cuda.synchronize()
        ctx.moe_decode_step_dev(0, L, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K,
                                d_out.data_ptr(), d_eo.data_ptr())
        ctx.sync()
        out, eo = d_out.cpu().numpy(), d_eo.cpu().numpy()
        assert np.isfinite(out).all()
        # (1) one launch over 40 layers == 40 launches
        s_out = torch.zeros(H, device="cuda")
        s_eo = torch.zeros(K, H, device="cuda")
        for l in range(L):
            ctx.moe_decode_dev(l, d_x.data_ptr() + l * H * 4, d_idx.data_ptr() + l * K * 4,
                               d_w.data_ptr() + l * K * 4, K, s_out.data_ptr(), s_eo.data_ptr())
            ctx.sync()
            assert np.array_equal(s_out.cpu().numpy(), out[l]), l
            assert np.array_equal(s_eo.cpu().numpy(), eo[l]), l
        # (2) the weighted sum in slot order, fp32 (shaders.metal:2213-2228)
        for l in range(L):
            acc = np.zeros(H, np.float32)
            for k in range(K):
                acc = acc + w[tok, l, k] * eo[l, k]
            assert rel_err(out[l], acc) < 1e-6, l
        # (3) the routed experts of three layers against the oracle on their own bytes
        for l in (0, 17, 39):
            mini = np.concatenate([blob[l, int(e)].cpu().numpy() for e in idx[tok, l]])
            ref, ref_eo = orc.moe_experts_forward(mini, x[l], np.arange(K, dtype=np.int32), w[tok, l],
                                                  H, I, 3, nthreads=8)
            assert_parity(eo[l], ref_eo, "expert_out layer %d" % l)
            assert_parity(out[l], ref, "layer %d" % l)


def test_full_chunk_equals_positions(full_store, orc):
    """512 positions x top-8 over all 256 experts of a layer (4096 pairs): every sampled position
    equals its per-position call within the bar, a repeat is bit-identical, and one position is
    checked against the oracle."""
    import torch
    from bench import zipf_routing
    ctx, blob, lo, _, _ = full_store
    M, layer = 512, 3
    rng = np.random.default_rng(8)
    idx, w = zipf_routing(rng, M, 1, E, K)
    idx, w = np.ascontiguousarray(idx[:, 0]), np.ascontiguousarray(w[:, 0])
    X = torch.randn(M, H).to(torch.bfloat16).to(torch.float32).numpy()
    out = ctx.moe_prefill(layer, X, idx, w)
    assert np.isfinite(out).all()
    assert np.array_equal(ctx.moe_prefill(layer, X, idx, w), out)
    # cover the hot experts' many items as well as the tail
    for m in list(range(0, M, 37)) + [M - 1]:
        single, _ = ctx.moe_decode(layer, X[m], idx[m], w[m])
        assert rel_err(out[m], single) < 1e-3 and cosine(out[m], single) > 0.99999, m
    m = 123
    mini = np.concatenate([blob[layer, int(e)].cpu().numpy() for e in idx[m]])
    ref, _ = orc.moe_experts_forward(mini, X[m], np.arange(K, dtype=np.int32), w[m], H, I, 3, nthreads=8)
    assert_parity(out[m], ref, "position %d" % m)


def test_full_chunk_bf16_entry_equals_positions(full_store, orc):
    """The same 512-position chunk handed over as bf16 bits (fm_moe_prefill_bf16: 16 positions per
    gate/up item, one matrix-core operand per value — the entry bench.py's prefill workload
    times): equal to the fp32 entry on the widened values within the bar, to per-position calls,
    and to the oracle on one position; a repeat is bit-identical."""
    import torch
    from bench import zipf_routing
    ctx, blob, lo, _, _ = full_store
    M, layer = 512, 5
    rng = np.random.default_rng(18)
    idx, w = zipf_routing(rng, M, 1, E, K)
    idx, w = np.ascontiguousarray(idx[:, 0]), np.ascontiguousarray(w[:, 0])
    Xb = torch.randn(M, H).to(torch.bfloat16)
    X = Xb.to(torch.float32).numpy()
    bits = Xb.view(torch.int16).numpy().view(np.uint16)
    out = ctx.moe_prefill_bf16(layer, bits, idx, w)
    assert np.isfinite(out).all()
    assert np.array_equal(ctx.moe_prefill_bf16(layer, bits, idx, w), out)
    wide = ctx.moe_prefill(layer, X, idx, w)
    for m in list(range(0, M, 29)) + [M - 1]:
        assert rel_err(out[m], wide[m]) < 1e-3 and cosine(out[m], wide[m]) > 0.99999, m
        single, _ = ctx.moe_decode(layer, X[m], idx[m], w[m])
        assert rel_err(out[m], single) < 1e-3 and cosine(out[m], single) > 0.99999, m
    m = 77
    mini = np.concatenate([blob[layer, int(e)].cpu().numpy() for e in idx[m]])
    ref, _ = orc.moe_experts_forward(mini, X[m], np.arange(K, dtype=np.int32), w[m], H, I, 3, nthreads=8)
    assert_parity(out[m], ref, "position %d" % m)


def test_lm_head_8bit_full_size(orc):
    """The 8-bit vocabulary projection at its real size, 248320 x 2048 (the streaming kernel of
    bench.py's lm_head workload): a few thousand sampled rows against the oracle, all outputs
    finite, and embedding rows bit for bit."""
    import torch
    from finchmoe_amd import FinchHip
    V, D = 248320, 2048
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(11)
    W = torch.empty(V * D, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
    s = torch.randn(V * (D // 64), device=dev, generator=gen).abs_() * (0.02 / 127.5)
    S = (s.view(torch.int32) >> 16).to(torch.int16)
    B = ((s * -127.5).view(torch.int32) >> 16).to(torch.int16)
    x = torch.randn(D, device=dev, generator=gen)
    out = torch.empty(V, device=dev)
    torch.cuda.synchronize()
    ctx = FinchHip(0)
    try:
        t = ctx.tensor_adopt(W.data_ptr(), S.data_ptr(), B.data_ptr(), V, D, 8)
        ctx.matvec_batch_dev([t], x.data_ptr(), [out.data_ptr()])
        ctx.sync()
        got = out.cpu().numpy()
        assert np.isfinite(got).all()
        rng = np.random.default_rng(6)
        rows = np.unique(np.concatenate([rng.integers(0, V, 3000), [0, 1, 2, 3, V - 4, V - 3, V - 2, V - 1]]))
        sel = torch.from_numpy(rows).to(dev)
        Wh = W.view(V, D)[sel].cpu().numpy()
        Sh = S.view(V, D // 64)[sel].cpu().numpy().view(np.uint16)
        Bh = B.view(V, D // 64)[sel].cpu().numpy().view(np.uint16)
        ref = orc.dequant_matvec(Wh.reshape(-1), Sh.reshape(-1), Bh.reshape(-1), x.cpu().numpy(), len(rows), D, 8)
        assert_parity(got[rows], ref, "sampled rows of the 8-bit vocabulary projection")
        ids = torch.tensor([5, V - 1], dtype=torch.int32, device=dev)
        emb = torch.empty(2, D, device=dev)
        ctx.embed_lookup_dev(t, ids.data_ptr(), 2, emb.data_ptr())
        ctx.sync()
        for i, tok in enumerate((5, V - 1)):
            k = int(np.searchsorted(rows, tok)) if tok in rows else None
            Wr = W.view(V, D)[tok].cpu().numpy()
            Sr = S.view(V, D // 64)[tok].cpu().numpy().view(np.uint16)
            Br = B.view(V, D // 64)[tok].cpu().numpy().view(np.uint16)
            _, w32 = orc.dequant_affine(Wr, Sr, Br, 1, D, 8)
            assert np.array_equal(emb[i].cpu().numpy().view(np.uint32), w32[0].view(np.uint32)), (tok, k)
    finally:
        ctx.close()


def test_full_chunk_4bit_equals_positions(orc):
    """The same 512-position chunk on one layer of 256 4-bit experts (453 MB): the grouped
    product against per-position calls, and one position against the oracle."""
    import torch
    from bench import fill_affine_layer, zipf_routing
    from finchmoe_amd import FinchHip
    dev = torch.device("cuda:0")
    lo = F.expert_layout(H, I, 4)
    es = lo["expert_size"]
    gen = torch.Generator(device=dev)
    gen.manual_seed(77)
    blob = torch.empty(1, E, es, dtype=torch.uint8, device=dev)
    fill_affine_layer(blob[0], lo, 4, gen)
    torch.cuda.synchronize()       # the context's stream does not wait for torch's
    ctx = FinchHip(0)
    try:
        ctx.experts_config(1, E, H, I, 64, 4, 0)
        ctx.experts_adopt_layer(0, blob[0].data_ptr(), E * es)
        M = 512
        idx, w = zipf_routing(np.random.default_rng(9), M, 1, E, K)
        idx, w = np.ascontiguousarray(idx[:, 0]), np.ascontiguousarray(w[:, 0])
        X = torch.randn(M, H).to(torch.bfloat16).to(torch.float32).numpy()
        out = ctx.moe_prefill(0, X, idx, w)
        assert np.isfinite(out).all()
        assert np.array_equal(ctx.moe_prefill(0, X, idx, w), out)
        for m in list(range(0, M, 41)) + [M - 1]:
            single, _ = ctx.moe_decode(0, X[m], idx[m], w[m])
            assert rel_err(out[m], single) < 1e-3 and cosine(out[m], single) > 0.99999, m
        m = 77
        mini = np.concatenate([blob[0, int(e)].cpu().numpy() for e in idx[m]])
        ref, _ = orc.moe_experts_forward(mini, X[m], np.arange(K, dtype=np.int32), w[m], H, I, 4, nthreads=8)
        assert_parity(out[m], ref, "position %d" % m)
    finally:
        ctx.close()
        del blob
        torch.cuda.empty_cache()


def test_full_step_without_expert_vectors_equals_with(full_store):
    """At the benchmark's size the launch that sums the experts in LDS (no buffer for the
    per-expert vectors) returns, bit for bit, what the launch with per-expert vectors and a
    combine phase returns — also when it accumulates, and twice in a row (activation sets)."""
    import torch
    from finchmoe_amd import binding as fb
    ctx, blob, lo, idx, w = full_store
    x = torch.randn(L, H, device="cuda", generator=torch.Generator(device="cuda").manual_seed(9))
    for tok, flags in ((0, 0), (1, fb.ACCUMULATE), (0, 0)):
        d_idx, d_w = torch.from_numpy(idx[tok]).cuda(), torch.from_numpy(w[tok]).cuda()
        base = torch.full((L, H), 0.25, device="cuda")
        want, got = base.clone(), base.clone()
        d_eo = torch.zeros(L, K, H, device="cuda")
        torch.cuda.synchronize()
        ctx.moe_decode_step_dev(0, L, x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K, want.data_ptr(),
                                d_eo.data_ptr(), flags)
        ctx.moe_decode_step_dev(0, L, x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K, got.data_ptr(),
                                None, flags)
        ctx.sync()
        assert torch.isfinite(got).all() and torch.equal(got, want), (tok, flags)


def test_full_gguf_step_equals_layer_calls_and_oracle(orc):
    """The GGUF store at the benchmark's size (40 layers x 256 experts, Q4_K gate/up and Q6_K
    down, 21.5 GB): the 40-layer step equals the 40 single-layer calls bit for bit, the weighted
    sum equals the per-expert outputs combined in slot order, and the routed experts of three
    layers equal the CPU oracle on their own bytes copied back."""
    import torch
    from bench import zipf_routing
    from finchmoe_amd import FinchHip
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    gsl, dsl = I * (H // 256) * 144, H * (I // 256) * 210      # bytes per expert: gate/up, down

    def slab(nblocks, bsz, d_off, n_d):
        t = torch.empty(nblocks, bsz, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
        d = (torch.randn(nblocks, n_d, device=dev, generator=gen).abs_() * 0.002).to(torch.float16)
        t[:, d_off:d_off + 2 * n_d] = d.view(torch.uint8)
        return t

    ctx = FinchHip(0)
    keep = []
    try:
        ctx.gguf_config(L, E, H, I)
        for l in range(L):
            g = slab(E * I * (H // 256), 144, 0, 2)
            u = slab(E * I * (H // 256), 144, 0, 2)
            d = slab(E * H * (I // 256), 210, 208, 1)
            keep.append((g, u, d))
            ctx.gguf_adopt_layer(l, g.data_ptr(), g.numel(), u.data_ptr(), u.numel(), d.data_ptr(), d.numel())
        idx, w = zipf_routing(np.random.default_rng(15), 1, L, E, K)
        idx, w = idx[0], w[0]
        x = np.random.default_rng(16).standard_normal((L, H)).astype(np.float32)
        d_x, d_idx, d_w = (torch.from_numpy(a).cuda() for a in (x, idx, w))
        d_out, d_eo = torch.zeros(L, H, device=dev), torch.zeros(L, K, H, device=dev)
        torch.cuda.synchronize()
        ctx.gguf_moe_decode_step_dev(0, L, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K,
                                     d_out.data_ptr(), d_eo.data_ptr())
        ctx.sync()
        out, eo = d_out.cpu().numpy(), d_eo.cpu().numpy()
        assert np.isfinite(out).all() and np.abs(out).max() > 0
        # the same step without the per-expert vectors as one launch (the library's own choice for
        # more than 13 layers is the three launches): the same bits, twice
        from finchmoe_amd import binding as fb
        try:
            ctx.set_kernel_forms(fb.FORM_GGUF_ONE_LAUNCH)
            for _ in range(2):
                d_one = torch.zeros(L, H, device=dev)
                torch.cuda.synchronize()
                ctx.gguf_moe_decode_step_dev(0, L, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K, d_one.data_ptr())
                ctx.sync()
                assert np.array_equal(d_one.cpu().numpy().view(np.uint32), out.view(np.uint32))
        finally:
            ctx.set_kernel_forms(0)
        d_dflt = torch.zeros(L, H, device=dev)
        torch.cuda.synchronize()
        ctx.gguf_moe_decode_step_dev(0, L, d_x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K, d_dflt.data_ptr())
        ctx.sync()
        assert np.array_equal(d_dflt.cpu().numpy().view(np.uint32), out.view(np.uint32))
        s_out, s_eo = torch.zeros(H, device=dev), torch.zeros(K, H, device=dev)
        for l in range(L):
            ctx.gguf_moe_decode_dev(l, d_x.data_ptr() + l * H * 4, d_idx.data_ptr() + l * K * 4,
                                    d_w.data_ptr() + l * K * 4, K, s_out.data_ptr(), s_eo.data_ptr())
            ctx.sync()
            assert np.array_equal(s_out.cpu().numpy(), out[l]), l
            assert np.array_equal(s_eo.cpu().numpy(), eo[l]), l
            acc = np.zeros(H, np.float32)
            for k in range(K):
                acc = acc + w[l, k] * eo[l, k]
            assert rel_err(out[l], acc) < 1e-6, l
        for l in (0, 21, 39):
            g, u, d = keep[l]
            mg = np.concatenate([g.view(E, gsl)[int(e)].cpu().numpy() for e in idx[l]])
            mu = np.concatenate([u.view(E, gsl)[int(e)].cpu().numpy() for e in idx[l]])
            md = np.concatenate([d.view(E, dsl)[int(e)].cpu().numpy() for e in idx[l]])
            ref, ref_eo = orc.moe_gguf_forward(mg, mu, md, x[l], np.arange(K, dtype=np.int32), w[l], H, I,
                                               nthreads=8)
            assert_parity(eo[l], ref_eo, "gguf expert_out layer %d" % l)
            assert_parity(out[l], ref, "gguf layer %d" % l)
    finally:
        ctx.close()
        del keep
        torch.cuda.empty_cache()
