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
        hip.layer_tail_dev(t, dev[0].data_ptr(), dev[1].data_ptr(), dev[2].data_ptr(), K,
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
