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
