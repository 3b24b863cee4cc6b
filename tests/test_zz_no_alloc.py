"""fm_moe_decode_step_noalloc_dev — the entry point that allocates nothing — against
fm_moe_decode_step_dev through the C ABI: bit for bit, on two calls in a row, the second with
a smaller input (the fixed scratch array keeps the first call's contents), plus the size limit.
Collected last (the file name sorts behind the other tests): it must pass alone in a fresh
process and after everything else."""
import numpy as np
import pytest

from finchmoe_amd import binding as fb
from finchmoe_amd import formats as F
from .conftest import assert_parity

pytestmark = pytest.mark.gpu

H, I, E, L = 2048, 512, 10, 6


def test_noalloc_entry_equals_the_allocating_one(orc):
    import torch
    from finchmoe_amd import FinchHip, FinchError
    rng = np.random.default_rng(99)
    blobs = [F.synth_expert_layer(rng, E, H, I, 3) for _ in range(L)]
    ctx = FinchHip(0)
    try:
        ctx.experts_config(L, E, H, I, 64, 3, fb.SCALE_BF16)
        for l, b in enumerate(blobs):
            ctx.experts_upload_layer(l, b)

        def inputs(n_layers, K, seed):
            r = np.random.default_rng(seed)
            x = r.standard_normal((n_layers, H)).astype(np.float32)
            idx = np.stack([orc.route(r.standard_normal(E).astype(np.float32), K)[0] for _ in range(n_layers)])
            w = np.stack([orc.normalize_weights(r.random(K).astype(np.float32)) for _ in range(n_layers)])
            return x, idx, w, [torch.from_numpy(a).cuda() for a in (x, idx, w)]

        # first call: all layers, K = 8; second call: fewer layers from another start, K = 5
        for (layer0, n_layers, K, seed) in ((0, L, 8, 1), (2, 3, 5, 2), (0, L, 8, 3)):
            x, idx, w, (dx, di, dw) = inputs(n_layers, K, seed)
            want = torch.zeros(n_layers, H, device="cuda")
            got = torch.full((n_layers, H), float("nan"), device="cuda")
            torch.cuda.synchronize()
            ctx.moe_decode_step_dev(layer0, n_layers, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), K,
                                    want.data_ptr())
            ctx.sync()
            ctx.moe_decode_step_noalloc_dev(layer0, n_layers, dx.data_ptr(), di.data_ptr(),
                                            dw.data_ptr(), K, got.data_ptr())
            ctx.sync()
            a, b = got.cpu().numpy(), want.cpu().numpy()
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (layer0, n_layers, K)
            ref, _ = orc.moe_experts_forward(blobs[layer0 + 1], x[1], idx[1], w[1], H, I, 3)
            assert_parity(a[1], ref, "no-alloc entry vs oracle")
        # accumulate flag, back to back without a sync in between
        x, idx, w, (dx, di, dw) = inputs(L, 8, 4)
        base = torch.randn(L, H, device="cuda")
        want, got = base.clone(), base.clone()
        torch.cuda.synchronize()
        ctx.moe_decode_step_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), 8, want.data_ptr(),
                                None, fb.ACCUMULATE)
        ctx.moe_decode_step_noalloc_dev(0, L, dx.data_ptr(), di.data_ptr(), dw.data_ptr(), 8,
                                        got.data_ptr(), fb.ACCUMULATE)
        ctx.sync()
        assert torch.equal(want, got)
    finally:
        ctx.close()
    # beyond the fixed array: a clear error, nothing launched
    big = FinchHip(0)
    try:
        n = 64                                   # 64 * 8 * 2560 * 4 B > 4 MiB
        big.experts_config(n, 1, H, I, 64, 3, fb.SCALE_BF16)
        blob = torch.zeros(big.expert_size(), dtype=torch.uint8, device="cuda")
        for l in range(n):
            big.experts_adopt_layer(l, blob.data_ptr(), blob.numel())
        z = torch.zeros(n * H, device="cuda")
        zi = torch.zeros(n * 8, dtype=torch.int32, device="cuda")
        with pytest.raises(FinchError) as e:
            big.moe_decode_step_noalloc_dev(0, n, z.data_ptr(), zi.data_ptr(), z.data_ptr(), 8, z.data_ptr())
        assert e.value.status == fb.ERR_ARG and "scratch" in str(e.value)
        big.moe_decode_step_noalloc_dev(0, 40, z.data_ptr(), zi.data_ptr(), z.data_ptr(), 8, z.data_ptr())
        big.sync()
    finally:
        big.close()
