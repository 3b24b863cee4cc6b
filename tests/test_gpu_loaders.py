"""Files in the reference's formats -> loaders -> C ABI -> results equal to the CPU oracle on the
same bytes."""
import numpy as np
import pytest

from finchmoe_amd import FinchHip, binding as fb, formats as F, loaders
from .conftest import assert_parity
from .test_host_loaders import write_dense, write_gguf

pytestmark = pytest.mark.gpu


def test_files_to_results(orc, tmp_path):
    rng = np.random.default_rng(11)
    Hh, Ii, E, K = 1024, 256, 6, 4
    ctx = FinchHip(0)
    try:
        # expert files
        blobs = [F.synth_expert_layer(rng, E, Hh, Ii, 3) for _ in range(2)]
        d = tmp_path / "packed_experts_3bit"
        d.mkdir()
        for l, b in enumerate(blobs):
            (d / ("layer_%02d.bin" % l)).write_bytes(b.tobytes())
        ctx.experts_config(2, E, Hh, Ii, 64, 3, 0)
        loaders.ExpertFiles(str(d), n_layers=2).upload(ctx)
        x = rng.standard_normal(Hh).astype(np.float32)
        idx, w = orc.route(rng.standard_normal(E).astype(np.float32), K)
        for l in range(2):
            out, _ = ctx.moe_decode(l, x, idx, w)
            assert_parity(out, orc.moe_experts_forward(blobs[l], x, idx, w, Hh, Ii, 3)[0], "layer %d" % l)
        # dense file
        t4 = F.synth_affine_tensor(rng, 512, Hh, 4)
        W4 = np.ascontiguousarray(t4[1]).view(np.uint32).reshape(512, -1)
        b, j = str(tmp_path / "model_weights_quant.bin"), str(tmp_path / "model_weights_quant.json")
        write_dense(b, j, {"model.layers.0.mlp.shared_expert.gate_proj.weight": ("q", W4, t4[2], t4[3], 4, 64)})
        df = loaders.DenseFile(b)
        t = df.register(ctx, "model.layers.0.mlp.shared_expert.gate_proj.weight")
        (got,) = ctx.matvec_batch([t], x, [512])
        assert_parity(got, orc.dequant_matvec(t4[1], t4[2], t4[3], x, 512, Hh, 4), "dense")
        # GGUF file
        g, u, dn = F.synth_gguf_layer(rng, E, Hh, Ii)
        path = str(tmp_path / "m.gguf")
        write_gguf(path, [("general.alignment", 4, 32)],
                   [("blk.0.ffn_gate_exps.weight", 12, [Hh, Ii, E], g.tobytes()),
                    ("blk.0.ffn_up_exps.weight", 12, [Hh, Ii, E], u.tobytes()),
                    ("blk.0.ffn_down_exps.weight", 14, [Ii, Hh, E], dn.tobytes())])
        gf = loaders.GgufFile(path)
        ne, hh, ii, types = gf.expert_geometry()
        ctx.gguf_config(1, ne, hh, ii, types)
        gf.upload_experts(ctx)
        out, _ = ctx.gguf_moe_decode(0, x, idx, w)
        assert_parity(out, orc.moe_gguf_forward(g, u, dn, x, idx, w, Hh, Ii)[0], "gguf")
    finally:
        ctx.close()


def test_c_host_loads_files_and_computes(orc, tmp_path):
    """The same three file kinds through the C host layer alone: finch_ops_load_expert_dir,
    finch_ops_open_dense + finch_ops_load_dense_tensor, finch_ops_open_gguf +
    finch_ops_load_gguf_experts, then the reference-named operators on what they loaded."""
    import ctypes as C
    L = loaders.lib()
    vp, i = C.c_void_p, C.c_int
    L.fast_dequant_matvec.argtypes = [vp, vp, vp, vp, vp, i, i, i, i]
    L.moe_experts_forward.argtypes = [i, vp, vp, vp, i, vp]
    L.gpu_gguf_experts_forward.argtypes = [i, vp, vp, vp, i, vp]
    L.finch_ops_last_error.restype = C.c_char_p
    rng = np.random.default_rng(12)
    Hh, Ii, E, K = 1024, 256, 6, 4
    assert L.finch_ops_init(0) == 0, L.finch_ops_last_error()
    try:
        blobs = [F.synth_expert_layer(rng, E, Hh, Ii, 3) for _ in range(3)]
        d = tmp_path / "packed_experts_3bit"
        d.mkdir()
        for l in (0, 2):                                  # layer 1 has no file: skipped
            (d / ("layer_%02d.bin" % l)).write_bytes(blobs[l].tobytes())
        assert L.finch_ops_config_experts(3, E, Hh, Ii, 3) == 0
        assert L.finch_ops_load_expert_dir(str(d).encode(), 3) == 2, loaders._err()
        x = rng.standard_normal(Hh).astype(np.float32)
        idx, w = orc.route(rng.standard_normal(E).astype(np.float32), K)
        for l in (0, 2):
            out = np.zeros(Hh, np.float32)
            assert L.moe_experts_forward(l, x.ctypes.data, idx.ctypes.data, w.ctypes.data, K, out.ctypes.data) == 1
            assert_parity(out, orc.moe_experts_forward(blobs[l], x, idx, w, Hh, Ii, 3)[0], "layer %d" % l)
        out = np.zeros(Hh, np.float32)
        assert L.moe_experts_forward(1, x.ctypes.data, idx.ctypes.data, w.ctypes.data, K, out.ctypes.data) == 0
        (d / "layer_01.bin").write_bytes(blobs[1].tobytes()[:-3])
        assert L.finch_ops_load_expert_dir(str(d).encode(), 3) < 0 and b"layer_01.bin" in L.finch_files_last_error()

        t4 = F.synth_affine_tensor(rng, 512, Hh, 4)
        W4 = np.ascontiguousarray(t4[1]).view(np.uint32).reshape(512, -1)
        b, j = str(tmp_path / "model_weights_quant.bin"), str(tmp_path / "model_weights_quant.json")
        name = "model.layers.0.mlp.shared_expert.gate_proj.weight"
        write_dense(b, j, {name: ("q", W4, t4[2], t4[3], 4, 64)})
        h = L.finch_ops_open_dense(b.encode(), None)
        assert h, loaders._err()
        assert L.finch_ops_load_dense_tensor(h, name.encode()) == 0, loaders._err()
        W, S, B = vp(), vp(), vp()
        od, idim, bits, gs = i(), i(), i(), i()
        assert L.finch_dense_quantized(h, name.encode(), C.byref(W), C.byref(S), C.byref(B), C.byref(od),
                                       C.byref(idim), C.byref(bits), C.byref(gs)) == 0
        got = np.zeros(512, np.float32)
        L.fast_dequant_matvec(W, S, B, x.ctypes.data, got.ctypes.data, od.value, idim.value, gs.value, bits.value)
        assert L.finch_ops_last_status() == 0, L.finch_ops_last_error()
        assert_parity(got, orc.dequant_matvec(t4[1], t4[2], t4[3], x, 512, Hh, 4), "dense")
        L.finch_ops_close_dense(h)

        g, u, dn = F.synth_gguf_layer(rng, E, Hh, Ii)
        path = str(tmp_path / "m.gguf")
        write_gguf(path, [], [("blk.1.ffn_gate_exps.weight", 12, [Hh, Ii, E], g.tobytes()),
                              ("blk.1.ffn_up_exps.weight", 12, [Hh, Ii, E], u.tobytes()),
                              ("blk.1.ffn_down_exps.weight", 14, [Ii, Hh, E], dn.tobytes())])
        gh = L.finch_ops_open_gguf(path.encode())
        assert gh, loaders._err()
        ne, hh, ii, types = i(), i(), i(), (C.c_int * 3)()
        assert L.finch_gguf_expert_geometry(gh, -1, C.byref(ne), C.byref(hh), C.byref(ii), types) == 0
        assert L.finch_ops_config_gguf_experts(2, ne.value, hh.value, ii.value, *types) == 0
        assert L.finch_ops_load_gguf_experts(gh, 2) == 1, loaders._err()
        L.finch_ops_close_gguf(gh)                         # the layer is resident: the file can go
        out = np.zeros(Hh, np.float32)
        assert L.gpu_gguf_experts_forward(1, x.ctypes.data, idx.ctypes.data, w.ctypes.data, K, out.ctypes.data) == 1
        assert_parity(out, orc.moe_gguf_forward(g, u, dn, x, idx, w, Hh, Ii)[0], "gguf")
    finally:
        L.finch_ops_shutdown()
