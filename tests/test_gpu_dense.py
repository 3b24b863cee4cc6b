"""GPU parity of the dense affine GEMV (GatedDeltaNet projections) against the CPU oracle."""
import numpy as np
import pytest

from finchmoe_amd import binding as fb
from finchmoe_amd import formats as F
from .conftest import assert_parity

pytestmark = pytest.mark.gpu


def _tensor(hip, rng, out_dim, in_dim, bits, dtype="bf16"):
    codes, W, S, B = F.synth_affine_tensor(rng, out_dim, in_dim, bits, dtype)
    sd = fb.SCALE_BF16 if dtype == "bf16" else fb.SCALE_FP16
    t = hip.tensor_register(W, S, B, out_dim, in_dim, bits, 64, sd)
    return t, (codes, W, S, B, sd)


def test_gdn_projections_4bit(hip, orc):
    """in_proj_qkv [8192,2048] + in_proj_z [4096,2048] from one x, then out_proj
    [2048,4096] (infer.m:8119-8122, 8500-8502)."""
    rng = np.random.default_rng(1)
    tq, q = _tensor(hip, rng, 8192, 2048, 4)
    tz, z = _tensor(hip, rng, 4096, 2048, 4)
    to, o = _tensor(hip, rng, 2048, 4096, 4)
    x = rng.standard_normal(2048).astype(np.float32)
    oq, oz = hip.matvec_batch([tq, tz], x, [8192, 4096])
    assert_parity(oq, orc.dequant_matvec(q[1], q[2], q[3], x, 8192, 2048, 4, nthreads=8), "qkv")
    assert_parity(oz, orc.dequant_matvec(z[1], z[2], z[3], x, 4096, 2048, 4, nthreads=8), "z")
    y = rng.standard_normal(4096).astype(np.float32)
    (oo,) = hip.matvec_batch([to], y, [2048])
    r, _ = assert_parity(oo, orc.dequant_matvec(o[1], o[2], o[3], y, 2048, 4096, 4, nthreads=8), "out_proj")
    assert r < 2e-5
    for t in (tq, tz, to):
        hip.tensor_release(t)


@pytest.mark.parametrize("bits,dtype,out_dim,in_dim", [
    (4, "bf16", 32, 2048), (4, "fp16", 100, 512), (8, "bf16", 256, 2048), (3, "bf16", 77, 1024),
    (4, "bf16", 5, 128), (8, "fp16", 33, 256), (4, "bf16", 64, 8192),
    (2, "bf16", 77, 1024), (2, "fp16", 100, 4096), (1, "bf16", 33, 192), (1, "fp16", 256, 2048), (2, "bf16", 3, 64)])
def test_matvec_shapes_and_widths(hip, orc, bits, dtype, out_dim, in_dim):
    """Ragged out_dim, small and large in_dim, every packing width (the legacy 1- and 2-bit
    widths of cpu_dequant_matvec, infer.m:1734, included), both scale types; codes and weights
    bit-exact, outputs within tolerance."""
    rng = np.random.default_rng(out_dim * 31 + in_dim + bits)
    t, (codes, W, S, B, sd) = _tensor(hip, rng, out_dim, in_dim, bits, dtype)
    gc, gw, gh = hip.dequant_tensor(t, out_dim, in_dim)
    rc, rw = orc.dequant_affine(W, S, B, out_dim, in_dim, bits, scale_dtype=sd)
    assert np.array_equal(gc, codes) and np.array_equal(gc, rc)
    assert np.array_equal(gw.view(np.uint32), rw.view(np.uint32))
    assert np.array_equal(gh, rw.astype(np.float16).view(np.uint16))
    x = rng.standard_normal(in_dim).astype(np.float32)
    (got,) = hip.matvec_batch([t], x, [out_dim])
    assert_parity(got, orc.dequant_matvec(W, S, B, x, out_dim, in_dim, bits, scale_dtype=sd), "matvec")
    # one-hot input returns a dequantized column
    e = np.zeros(in_dim, np.float32)
    e[in_dim // 2 + 3] = 1.0
    (col,) = hip.matvec_batch([t], e, [out_dim])
    assert np.allclose(col, rw[:, in_dim // 2 + 3], rtol=1e-6, atol=1e-9)
    hip.tensor_release(t)


@pytest.mark.parametrize("bits,dtype,out_dim,in_dim", [
    (4, "bf16", 8192, 4096), (3, "bf16", 8192, 2048), (4, "fp16", 16384, 1024),
    (3, "fp16", 32768, 512), (8, "bf16", 16384, 2048), (8, "fp16", 32768, 1024), (8, "bf16", 65536, 512)])
def test_streaming_kernel_shapes(hip, orc, bits, dtype, out_dim, in_dim):
    """Launches large enough for the streaming kernel (a wave step for every wave of the
    chip): two column slabs at in_dim 4096, every lanes-per-row specialisation, both widths
    and scale types; M positions equal the single call bitwise."""
    rng = np.random.default_rng(out_dim + in_dim + bits)
    t, (codes, W, S, B, sd) = _tensor(hip, rng, out_dim, in_dim, bits, dtype)
    X = rng.standard_normal((2, in_dim)).astype(np.float32)
    (got,) = hip.matvec_batch([t], X[0], [out_dim])
    ref = orc.dequant_matvec(W, S, B, X[0], out_dim, in_dim, bits, scale_dtype=sd, nthreads=8)
    r, _ = assert_parity(got, ref, "matvec")
    assert r < 2e-5, r
    out = hip.matvec_prefill(t, X, out_dim)
    assert np.array_equal(out[0], got)
    assert_parity(out[1], orc.dequant_matvec(W, S, B, X[1], out_dim, in_dim, bits,
                                             scale_dtype=sd, nthreads=8), "position 1")
    hip.tensor_release(t)


def test_matvec_prefill_positions(hip, orc):
    """M-position clone (dequant_matvec_4bit_prefill): every position equals the single call."""
    rng = np.random.default_rng(3)
    t, (codes, W, S, B, sd) = _tensor(hip, rng, 512, 2048, 4)
    X = rng.standard_normal((8, 2048)).astype(np.float32)
    out = hip.matvec_prefill(t, X, 512)
    for m in range(8):
        (single,) = hip.matvec_batch([t], X[m], [512])
        assert np.array_equal(out[m], single)
        assert_parity(out[m], orc.dequant_matvec(W, S, B, X[m], 512, 2048, 4), "pos %d" % m)
    hip.tensor_release(t)


def test_low_widths_in_a_batch_and_over_positions(hip, orc):
    """2-bit tensors in one batch with a 4-bit one (separate launches, one call), and a 1-bit
    tensor against several positions: each position equals the single call bitwise."""
    rng = np.random.default_rng(40)
    t2a, a = _tensor(hip, rng, 96, 1024, 2)
    t2b, b = _tensor(hip, rng, 40, 1024, 2)
    t4, c4 = _tensor(hip, rng, 64, 1024, 4)
    x = rng.standard_normal(1024).astype(np.float32)
    oa, ob, o4 = hip.matvec_batch([t2a, t2b, t4], x, [96, 40, 64])
    assert_parity(oa, orc.dequant_matvec(a[1], a[2], a[3], x, 96, 1024, 2), "2-bit a")
    assert_parity(ob, orc.dequant_matvec(b[1], b[2], b[3], x, 40, 1024, 2), "2-bit b")
    assert_parity(o4, orc.dequant_matvec(c4[1], c4[2], c4[3], x, 64, 1024, 4), "4-bit")
    t1, d = _tensor(hip, rng, 50, 512, 1)
    X = rng.standard_normal((20, 512)).astype(np.float32)
    out = hip.matvec_prefill(t1, X, 50)
    for m in (0, 7, 19):
        (one,) = hip.matvec_batch([t1], X[m], [50])
        assert np.array_equal(out[m], one)
        assert_parity(out[m], orc.dequant_matvec(d[1], d[2], d[3], X[m], 50, 512, 1), "1-bit position %d" % m)
    for t in (t2a, t2b, t4, t1):
        hip.tensor_release(t)


def test_kernel_forms_override(hip, orc):
    """fm_set_kernel_forms: the plain kernel for a shape that streams by default agrees with the
    oracle too; with the dense GEMM switched off a 40-position call equals the one-position
    calls bitwise; unknown flags are refused; 0 restores the default."""
    from finchmoe_amd import FinchError
    rng = np.random.default_rng(41)
    t, (codes, W, S, B, sd) = _tensor(hip, rng, 8192, 2048, 4)
    X = rng.standard_normal((40, 2048)).astype(np.float32)
    ref = orc.dequant_matvec(W, S, B, X[0], 8192, 2048, 4, nthreads=8)
    (dflt,) = hip.matvec_batch([t], X[0], [8192])
    try:
        hip.set_kernel_forms(fb.FORM_PLAIN_DENSE)
        (plain,) = hip.matvec_batch([t], X[0], [8192])
        assert_parity(plain, ref, "plain kernel")
        hip.set_kernel_forms(fb.FORM_NO_DENSE_GEMM)
        out = hip.matvec_prefill(t, X, 8192)
        for m in (0, 17, 39):
            (one,) = hip.matvec_batch([t], X[m], [8192])
            assert np.array_equal(out[m], one), m
        with pytest.raises(FinchError):
            hip.set_kernel_forms(1 << 9)
    finally:
        hip.set_kernel_forms(0)
    (again,) = hip.matvec_batch([t], X[0], [8192])
    assert np.array_equal(again, dflt)
    assert_parity(dflt, ref, "streaming kernel")
    hip.tensor_release(t)


def test_mixed_batch_and_errors(hip, orc):
    rng = np.random.default_rng(4)
    t4, a = _tensor(hip, rng, 64, 2048, 4)
    t8, b = _tensor(hip, rng, 32, 2048, 8)
    x = rng.standard_normal(2048).astype(np.float32)
    o4, o8 = hip.matvec_batch([t4, t8], x, [64, 32])    # mixed widths: split into two launches
    assert_parity(o4, orc.dequant_matvec(a[1], a[2], a[3], x, 64, 2048, 4), "4-bit")
    assert_parity(o8, orc.dequant_matvec(b[1], b[2], b[3], x, 32, 2048, 8), "8-bit")
    from finchmoe_amd import FinchError
    t5, _ = _tensor(hip, rng, 16, 512, 4)
    with pytest.raises(FinchError):
        hip.matvec_batch([t4, t5], x, [64, 16])           # in_dim mismatch
    with pytest.raises(FinchError):
        hip.matvec_batch([12345], x, [64])
    with pytest.raises(FinchError) as e:
        hip.tensor_register(a[1], a[2], a[3], 64, 2000, 4)
    assert e.value.status == fb.ERR_UNSUPPORTED
    for t in (t4, t8, t5):
        hip.tensor_release(t)


@pytest.mark.parametrize("bits,dtype", [(8, "bf16"), (4, "bf16"), (4, "fp16")])
def test_embedding_lookup_is_the_dequantized_row(hip, orc, bits, dtype):
    """embed_lookup (infer.m:5664-5722): the row of a token, bit for bit the oracle's dequant of
    that row; ids from device memory, an id outside the table gives zeros."""
    import torch
    rng = np.random.default_rng(50 + bits)
    vocab, hidden = 1000, 2048
    _, W, S, B = F.synth_affine_tensor(rng, vocab, hidden, bits, dtype)
    sd = fb.SCALE_BF16 if dtype == "bf16" else fb.SCALE_FP16
    t = hip.tensor_register(W, S, B, vocab, hidden, bits, scale_dtype=sd)
    try:
        _, ref32 = orc.dequant_affine(W, S, B, vocab, hidden, bits, scale_dtype=sd)
        for tok in (0, 1, 517, vocab - 1):
            got = hip.embed_lookup(t, tok, hidden)
            assert np.array_equal(got.view(np.uint32), ref32[tok].view(np.uint32)), tok
        ids = np.array([3, 999, 3, -1, vocab, 42], np.int32)
        d_ids = torch.from_numpy(ids).cuda()
        d_out = torch.full((len(ids), hidden), 7.0, device="cuda")
        hip.embed_lookup_dev(t, d_ids.data_ptr(), len(ids), d_out.data_ptr())
        hip.sync()
        out = d_out.cpu().numpy()
        for i, tok in enumerate(ids):
            want = ref32[tok] if 0 <= tok < vocab else np.zeros(hidden, np.float32)
            assert np.array_equal(out[i].view(np.uint32), want.view(np.uint32)), (i, tok)
    finally:
        hip.tensor_release(t)


@pytest.mark.parametrize("bits,dtype,out_dim,in_dim,M", [
    (4, "bf16", 512, 2048, 64), (4, "bf16", 256, 4096, 40), (4, "fp16", 128, 2048, 33),
    (3, "bf16", 192, 2048, 100), (4, "bf16", 64, 8192, 32), (4, "bf16", 128, 2048, 16),
    (4, "bf16", 2048, 512, 40), (3, "fp16", 512, 512, 33)])
def test_dense_prefill_gemm_matches_positions(hip, orc, bits, dtype, out_dim, in_dim, M):
    """From 16 positions on, a dense 3-/4-bit tensor with in_dim 512 or a multiple of 2048 runs on
    the matrix cores (one column pass per 2048 columns): every position against the oracle's GEMV and
    against the one-position call."""
    rng = np.random.default_rng(out_dim + in_dim + M)
    t, (codes, W, S, B, sd) = _tensor(hip, rng, out_dim, in_dim, bits, dtype)
    try:
        X = rng.standard_normal((M, in_dim)).astype(np.float32)
        X[3] *= 1e-3
        X[5] *= 300.0
        out = hip.matvec_prefill(t, X, out_dim)
        assert out.shape == (M, out_dim) and np.isfinite(out).all()
        for m in range(M):
            (single,) = hip.matvec_batch([t], X[m], [out_dim])
            assert_parity(out[m], single, "position %d vs one-position call" % m)
        for m in (0, 3, 5, M - 1):
            ref = orc.dequant_matvec(W, S, B, X[m], out_dim, in_dim, bits, scale_dtype=sd, nthreads=8)
            assert_parity(out[m], ref, "position %d vs oracle" % m)
        assert np.array_equal(hip.matvec_prefill(t, X, out_dim), out)
    finally:
        hip.tensor_release(t)


def test_dense_prefill_batch_shares_the_prepared_input(hip, orc):
    """Two tensors of the same width (and a third of another) against the same positions in one
    call equal the single-tensor calls bit for bit."""
    import torch
    rng = np.random.default_rng(77)
    M = 48
    ta, _ = _tensor(hip, rng, 256, 2048, 4)
    tb, _ = _tensor(hip, rng, 128, 2048, 4)
    tc, _ = _tensor(hip, rng, 64, 2048, 3)
    td, _ = _tensor(hip, rng, 96, 2048, 8)          # no matrix-core form: one GEMV per position
    try:
        X = rng.standard_normal((M, 2048)).astype(np.float32)
        d_X = torch.from_numpy(X).cuda()
        dims = (256, 128, 64, 96)
        outs = [torch.zeros(M, d, device="cuda") for d in dims]
        hip.matvec_prefill_batch_dev([ta, tb, tc, td], d_X.data_ptr(), [o.data_ptr() for o in outs], M)
        hip.sync()
        for t, d, o in zip((ta, tb, tc, td), dims, outs):
            assert np.array_equal(o.cpu().numpy(), hip.matvec_prefill(t, X, d)), d
    finally:
        for t in (ta, tb, tc, td):
            hip.tensor_release(t)


@pytest.mark.parametrize("out_dim,in_dim", [(32, 2048), (256, 2048), (1, 2048), (7, 100), (33, 4096)])
def test_raw_bf16_matvec(hip, orc, out_dim, in_dim):
    """Tensors registered without scales and biases are unquantized BF16 [out][in]
    (cpu_dequant_matvec's scales == NULL branch, infer.m:1689-1701)."""
    rng = np.random.default_rng(out_dim * 7 + in_dim)
    W = F.bf16_trunc(rng.standard_normal((out_dim, in_dim)).astype(np.float32) * np.float32(0.1))
    t = hip.tensor_register(W, None, None, out_dim, in_dim, bits=0)
    x = rng.standard_normal(in_dim).astype(np.float32)
    (out,) = hip.matvec_batch([t], x, [out_dim])
    ref = orc.dequant_matvec(W, None, None, x, out_dim, in_dim, 0)
    want = F.bf16_to_f32(W).astype(np.float64) @ x.astype(np.float64)
    scale = max(float(np.max(np.abs(want))), 1e-30)
    assert np.max(np.abs(out - ref)) <= 1e-3 * scale and np.max(np.abs(out - want)) <= 1e-5 * scale
    # M positions equal the single calls bit for bit
    X = rng.standard_normal((5, in_dim)).astype(np.float32)
    om = hip.matvec_prefill(t, X, out_dim)
    for m in range(5):
        (single,) = hip.matvec_batch([t], X[m], [out_dim])
        assert np.array_equal(om[m], single)
    from finchmoe_amd import FinchError
    with pytest.raises(FinchError) as e:
        hip.dequant_tensor(t, out_dim, in_dim)
    assert e.value.status == fb.ERR_UNSUPPORTED
    hip.tensor_release(t)


def test_raw_bf16_in_a_mixed_batch(hip, orc):
    """One fm_matvec_batch call over 4-bit and BF16 tensors that share x."""
    rng = np.random.default_rng(77)
    t4, a = _tensor(hip, rng, 128, 2048, 4)
    Wb = F.bf16_trunc(rng.standard_normal((32, 2048)).astype(np.float32) * np.float32(0.1))
    tb = hip.tensor_register(Wb, None, None, 32, 2048)
    t4b, c = _tensor(hip, rng, 64, 2048, 4)
    x = rng.standard_normal(2048).astype(np.float32)
    o1, o2, o3 = hip.matvec_batch([t4, tb, t4b], x, [128, 32, 64])
    assert_parity(o1, orc.dequant_matvec(a[1], a[2], a[3], x, 128, 2048, 4), "4-bit first")
    assert_parity(o2, orc.dequant_matvec(Wb, None, None, x, 32, 2048, 0), "BF16")
    assert_parity(o3, orc.dequant_matvec(c[1], c[2], c[3], x, 64, 2048, 4), "4-bit last")
    for t in (t4, tb, t4b):
        hip.tensor_release(t)


def test_mixed_widths_in_one_batch_equal_separate_calls(hip, orc):
    """The routing batch of a layer — 8-bit router and shared-gate score, 4-bit shared gate/up,
    one x (finchmoe/infer.m:9285-9300) — goes out as one launch; every output equals, bit for
    bit, the tensor's own call, and the oracle within the bar.  A 3-bit tensor joins too."""
    rng = np.random.default_rng(77)
    Hh = 2048
    shapes = [(256, 8), (1, 8), (512, 4), (512, 4), (96, 3)]
    tens, handles = [], []
    for rows, bits in shapes:
        t = F.synth_affine_tensor(rng, rows, Hh, bits)
        tens.append(t)
        handles.append(hip.tensor_register(t[1], t[2], t[3], rows, Hh, bits))
    x = rng.standard_normal(Hh).astype(np.float32)
    outs = hip.matvec_batch(handles, x, [r for r, _ in shapes])
    for (rows, bits), t, h, got in zip(shapes, tens, handles, outs):
        (alone,) = hip.matvec_batch([h], x, [rows])
        assert np.array_equal(got, alone), (rows, bits)
        assert_parity(got, orc.dequant_matvec(t[1], t[2], t[3], x, rows, Hh, bits), "%d rows at %d bits" % (rows, bits))
    for h in handles:
        hip.tensor_release(h)


def test_gdn_set_is_one_launch_with_riders(hip, orc):
    """The reference's four-spec batch {qkv 8192, z 4096, b 32, a 32} on one x
    (finchmoe/infer.m:8118-8122): the two raw-BF16 tensors ride along in the streaming launch
    of the 4-bit ones.  Every output equals, bit for bit, what the launches without riders give,
    and the oracle within the bar."""
    rng = np.random.default_rng(78)
    Hh = 2048
    q4 = [F.synth_affine_tensor(rng, rows, Hh, 4) for rows in (8192, 4096)]
    raw = [F.bf16_trunc(rng.standard_normal((32, Hh)).astype(np.float32) * np.float32(0.1)) for _ in range(2)]
    hs = [hip.tensor_register(t[1], t[2], t[3], rows, Hh, 4) for t, rows in zip(q4, (8192, 4096))]
    hs += [hip.tensor_register(w, None, None, 32, Hh) for w in raw]
    dims = [8192, 4096, 32, 32]
    x = rng.standard_normal(Hh).astype(np.float32)
    outs = hip.matvec_batch(hs, x, dims)
    # the 4-bit pair without riders (same kernel), the raw tensors on their own
    for got, want in zip(outs[:2], hip.matvec_batch(hs[:2], x, dims[:2])):
        assert np.array_equal(got, want)
    for h, got in zip(hs[2:], outs[2:]):
        (alone,) = hip.matvec_batch([h], x, [32])
        assert np.array_equal(got, alone)
    for t, rows, got in zip(q4, (8192, 4096), outs[:2]):
        assert_parity(got, orc.dequant_matvec(t[1], t[2], t[3], x, rows, Hh, 4), "%d rows" % rows)
    for w, got in zip(raw, outs[2:]):
        assert_parity(got, orc.dequant_matvec(w, None, None, x, 32, Hh, 0), "raw BF16")
    for h in hs:
        hip.tensor_release(h)
