"""Readers of the reference's file formats (finchmoe_amd/loaders.py) on synthetic files written
here in the formats the reference's writers and readers define (quantize_non_experts.py:365-386,
infer.m:727-786 for the manifest; infer.m:1025-1247 for GGUF; repack_experts.py:349-351 for the
expert files).  No GPU: upload calls go to a recording stand-in."""
import json
import struct

import numpy as np
import pytest

from finchmoe_amd import formats as F
from finchmoe_amd import loaders


class _Recorder:
    def __init__(self, expert_size=0, n_experts=0):
        self._es, self.n_experts, self.calls = expert_size, n_experts, []

    def expert_size(self):
        return self._es

    def experts_upload_layer(self, layer, blob):
        self.calls.append(("experts", layer, np.array(blob)))

    def gguf_upload_layer(self, layer, g, u, d):
        self.calls.append(("gguf", layer, np.array(g), np.array(u), np.array(d)))

    def tensor_register(self, W, S, B, out_dim, in_dim, bits, gs):
        self.calls.append(("tensor", np.array(W), np.array(S), np.array(B), out_dim, in_dim, bits, gs))
        return len(self.calls) - 1


def write_dense(path_bin, path_json, tensors, align=64):
    """tensors: name -> ("q", W u32 2-D, S, B, bits, gs) or ("bf16", u16 array)."""
    manifest = {"model": "synthetic", "tensors": {}}
    off = 0
    with open(path_bin, "wb") as f:
        def put(name, data, shape, dtype, bits=None, gs=None):
            nonlocal off
            pad = (-off) % align
            f.write(b"\0" * pad)
            off += pad
            f.write(data)
            e = {"offset": off, "size": len(data), "shape": list(shape), "dtype": dtype}
            if bits:
                e["bits"], e["group_size"] = bits, gs
            manifest["tensors"][name] = e
            off += len(data)
        for name, t in tensors.items():
            if t[0] == "q":
                _, W, S, B, bits, gs = t
                base = name[:-len(".weight")]
                put(name, W.tobytes(), W.shape, "U32", bits, gs)
                put(base + ".scales", S.tobytes(), S.shape, "BF16", bits, gs)
                put(base + ".biases", B.tobytes(), B.shape, "BF16", bits, gs)
            else:
                put(name, t[1].tobytes(), t[1].shape, "BF16")
    with open(path_json, "w") as f:
        json.dump(manifest, f)


def _gstr(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def write_gguf(path, kv, tensors, alignment=32):
    """kv: list of (key, type id, value); tensors: list of (name, ggml type, dims, bytes)."""
    def val(vt, v):
        fmt = {0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 6: "f", 7: "?", 10: "Q", 11: "q", 12: "d"}
        if vt in fmt:
            return struct.pack("<" + fmt[vt], v)
        if vt == 8:
            return _gstr(v)
        at, items = v
        return struct.pack("<IQ", at, len(items)) + b"".join(val(at, x) for x in items)
    head = b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(kv))
    for k, vt, v in kv:
        head += _gstr(k) + struct.pack("<I", vt) + val(vt, v)
    offs, cur = [], 0
    for _, _, _, data in tensors:
        cur = (cur + alignment - 1) // alignment * alignment
        offs.append(cur)
        cur += len(data)
    for (name, gt, dims, _), off in zip(tensors, offs):
        head += _gstr(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", gt, off)
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * ((-len(head)) % alignment))
        pos = 0
        for (_, _, _, data), off in zip(tensors, offs):
            f.write(b"\0" * (off - pos))
            f.write(data)
            pos = off + len(data)


def test_dense_manifest_roundtrip(tmp_path):
    rng = np.random.default_rng(1)
    t4 = F.synth_affine_tensor(rng, 24, 256, 4)
    t8 = F.synth_affine_tensor(rng, 5, 128, 8)
    norm = rng.integers(0, 65536, 64).astype(np.uint16)
    W4 = np.ascontiguousarray(t4[1]).view(np.uint32).reshape(24, -1)
    W8 = np.ascontiguousarray(t8[1]).view(np.uint32).reshape(5, -1)
    b, j = str(tmp_path / "model_weights_quant.bin"), str(tmp_path / "model_weights_quant.json")
    write_dense(b, j, {
        "model.layers.0.linear_attn.in_proj_qkv.weight": ("q", W4, t4[2], t4[3], 4, 64),
        "model.layers.0.input_layernorm.weight": ("bf16", norm),
        "model.layers.0.mlp.gate.weight": ("q", W8, t8[2], t8[3], 8, 64)})
    d = loaders.DenseFile(b)
    assert d.model == "synthetic" and len(d.tensors) == 7
    assert all(t["offset"] % 64 == 0 for t in d.tensors.values())
    W, S, B, od, idim, bits, gs = d.quantized("model.layers.0.linear_attn.in_proj_qkv.weight")
    assert (od, idim, bits, gs) == (24, 256, 4, 64)
    assert np.array_equal(W, W4) and np.array_equal(S, t4[2]) and np.array_equal(B, t4[3])
    W, S, B, od, idim, bits, gs = d.quantized("model.layers.0.mlp.gate.weight")
    assert (od, idim, bits) == (5, 128, 8) and np.array_equal(W, W8)
    assert np.array_equal(d.raw("model.layers.0.input_layernorm.weight", np.uint16), norm)
    rec = _Recorder()
    h = d.register(rec, "model.layers.0.mlp.gate.weight")
    assert rec.calls[h][4:] == (5, 128, 8, 64)
    with pytest.raises(ValueError):
        d.quantized("model.layers.0.input_layernorm.weight")
    d.close()
    with open(j, "w") as f:
        json.dump({"no_tensors": {}}, f)
    with pytest.raises(ValueError):
        loaders.DenseFile(b)


def test_gguf_directory_and_expert_tensors(tmp_path):
    rng = np.random.default_rng(2)
    E, Hh, Ii = 3, 512, 256
    layers = {l: F.synth_gguf_layer(rng, E, Hh, Ii) for l in (0, 2)}
    f32 = rng.standard_normal(7).astype(np.float32)
    tensors = [("token_embd.weight", 0, [7], f32.tobytes())]
    for l, (g, u, d) in layers.items():
        tensors += [("blk.%d.ffn_gate_exps.weight" % l, 12, [Hh, Ii, E], g.tobytes()),
                    ("blk.%d.ffn_down_exps.weight" % l, 14, [Ii, Hh, E], d.tobytes()),
                    ("blk.%d.ffn_up_exps.weight" % l, 12, [Hh, Ii, E], u.tobytes())]
    tensors.append(("blk.1.ffn_gate_exps.weight", 12, [Hh, Ii, E], layers[0][0].tobytes()))  # incomplete layer
    kv = [("general.architecture", 8, "qwen"), ("general.alignment", 4, 64), ("x.f", 6, 1.5),
          ("x.flag", 7, True), ("x.big", 10, 1 << 40), ("tokenizer.tokens", 9, (8, ["a", "bc", ""])),
          ("x.arr", 9, (4, [1, 2, 3])), ("x.i8", 1, -3), ("x.f64", 12, 2.25)]
    path = str(tmp_path / "model.gguf")
    write_gguf(path, kv, tensors, alignment=64)
    gf = loaders.GgufFile(path)
    assert gf.version == 3 and gf.alignment == 64 and gf.data_off % 64 == 0
    assert gf.kv["tokenizer.tokens"] == ["a", "bc", ""] and gf.kv["x.arr"] == [1, 2, 3]
    assert gf.kv["x.big"] == 1 << 40 and gf.kv["x.i8"] == -3 and gf.kv["x.flag"] is True
    assert gf.expert_layers() == [0, 2]
    assert gf.expert_geometry() == (E, Hh, Ii, (12, 12, 14))
    assert gf.row_bytes("blk.0.ffn_gate_exps.weight") == Hh // 256 * 144
    assert gf.row_bytes("blk.0.ffn_down_exps.weight") == Ii // 256 * 210
    gt, dims, data = gf.tensor_bytes("blk.2.ffn_down_exps.weight")
    assert gt == 14 and dims == [Ii, Hh, E] and np.array_equal(data, layers[2][2])
    assert np.array_equal(gf.tensor_bytes("token_embd.weight")[2].view(np.float32), f32)
    rec = _Recorder()
    gf.upload_experts(rec)
    assert [c[1] for c in rec.calls] == [0, 2]
    for c in rec.calls:
        for got, want in zip(c[2:], layers[c[1]]):
            assert np.array_equal(got, want)
    gf.close()
    bad = str(tmp_path / "bad.gguf")
    with open(bad, "wb") as f:
        f.write(b"GGML" + b"\0" * 64)
    with pytest.raises(ValueError):
        loaders.GgufFile(bad)


def test_expert_files(tmp_path):
    rng = np.random.default_rng(3)
    lo = F.expert_layout(256, 128, 3)
    E = 4
    blobs = [F.synth_expert_layer(rng, E, 256, 128, 3) for _ in range(2)]
    d = tmp_path / "packed_experts_3bit"
    d.mkdir()
    for l, b in enumerate(blobs):
        (d / ("layer_%02d.bin" % l)).write_bytes(b.tobytes())
    rec = _Recorder(lo["expert_size"], E)
    loaders.ExpertFiles(str(d), n_layers=2).upload(rec)
    assert [c[1] for c in rec.calls] == [0, 1]
    assert all(np.array_equal(c[2], b.reshape(-1)) for c, b in zip(rec.calls, blobs))
    (d / "layer_01.bin").write_bytes(blobs[1].tobytes()[:-1])
    with pytest.raises(ValueError):
        loaders.ExpertFiles(str(d), n_layers=2).upload(_Recorder(lo["expert_size"], E))
