"""The C readers of the reference's file formats and the C quantizer (finchmoe_amd/host/finch_files.c,
reached through finchmoe_amd/loaders.py) on synthetic files written here in the formats the
reference's writers and readers define (quantize_non_experts.py:365-386, infer.m:727-786 for the
manifest; infer.m:1025-1247 for GGUF; repack_experts.py:349-351 for the expert files), and on the
committed quantizer vectors.  No GPU: upload calls go to a recording stand-in."""
import os
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
    # every value type above was stepped over correctly, or the names below would be garbage
    assert len(gf.infos) == len(tensors) and list(gf.infos) == [t[0] for t in tensors]
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


# ---- quantizer (product code, not the oracle) ----------------------------------------------

def _golden():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "quantizer_vectors.npz")
    return np.load(path, allow_pickle=False)


@pytest.mark.parametrize("key,bits", [("pack3", 3), ("pack4", 4), ("q3", 3), ("qm4", 4), ("qm8", 8),
                                      ("qne4", 4), ("qne8", 8)])
def test_c_quantizer_reproduces_reference_vectors(key, bits):
    """Packed bytes, scales and biases bit for bit against what the reference's four quantizers
    wrote for the committed inputs (tests/golden/make_quantizer_vectors.py): exact .5 ties,
    clamped scales, negative ranges."""
    g = _golden()
    packed, S, B = loaders.quantize_affine_pack(g["w"], bits)
    assert np.array_equal(packed, g[key + "_w"]), key
    assert np.array_equal(S, g[key + "_s"]) and np.array_equal(B, g[key + "_b"]), key


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_c_quantizer_equals_oracle_on_random_tensors(orc, bits):
    rng = np.random.default_rng(bits)
    w = (rng.standard_normal((40, 512)) * rng.uniform(1e-3, 3, (40, 1))).astype(np.float32)
    w[3] = 0.25                                   # constant rows: the scale clamp
    w[4, :64] = np.arange(64, dtype=np.float32)   # exact ties at every other code for 3 bits
    packed, S, B = loaders.quantize_affine_pack(w, bits)
    codes, So, Bo = orc.quantize_affine(w, bits)
    want = np.ascontiguousarray(F.pack_codes(codes, bits)).view(np.uint8).reshape(40, -1)
    assert np.array_equal(packed, want) and np.array_equal(S, So) and np.array_equal(B, Bo)


def test_c_quantizer_rejects_what_it_cannot_pack():
    w = np.zeros((2, 96), np.float32)
    for bits, gs in ((5, 32), (4, 64), (3, 36)):       # bits, 96 % 64, 36 % 8
        with pytest.raises(ValueError):
            loaders.quantize_affine_pack(w[:, :36] if gs == 36 else w, bits, gs)


def test_quantize_expert_lays_out_the_blob(orc):
    rng = np.random.default_rng(9)
    Hh, Ii = 256, 128
    gate, up = (rng.standard_normal((Ii, Hh)).astype(np.float32) for _ in range(2))
    down = rng.standard_normal((Hh, Ii)).astype(np.float32)
    for bits in (3, 4):
        blob = loaders.quantize_expert(gate, up, down, bits)
        lo = F.expert_layout(Hh, Ii, bits)
        assert blob.size == lo["expert_size"]
        v = F.expert_views(blob, 0, Hh, Ii, bits)
        for name, w in (("gate", gate), ("up", up), ("down", down)):
            packed, S, B = loaders.quantize_affine_pack(w, bits)
            assert np.array_equal(v[name][0], packed.reshape(-1))
            assert np.array_equal(v[name][1], S) and np.array_equal(v[name][2], B)
        # and it computes: the oracle's expert forward on the blob equals the one on the parts
        x = rng.standard_normal(Hh).astype(np.float32)
        idx, wts = np.array([0], np.int32), np.array([1.0], np.float32)
        got = orc.moe_experts_forward(blob.reshape(1, -1), x, idx, wts, Hh, Ii, bits)[0]
        assert np.all(np.isfinite(got)) and np.any(got != 0)


# ---- the C parsers on malformed and awkward input -------------------------------------------

def test_manifest_parser_edge_cases(tmp_path):
    b, j = str(tmp_path / "w.bin"), str(tmp_path / "w.json")
    with open(b, "wb") as f:
        f.write(bytes(range(256)))
    # escapes in names, nested values to skip, null bits, exponent numbers, keys in any order
    text = (r'{"extra": [1, {"a": [true, false, null, "x\"y"]}], "model": "m\u00e9\/x", '
            r'"tensors": {"a\"b": {"dtype": "BF16", "shape": [4, 2], "size": 16, "offset": 6.4e1, "bits": null},'
            r' "t": {"offset": 0, "size": 256, "shape": [], "dtype": "F32", "zzz": {"k": []}}}}')
    with open(j, "w") as f:
        f.write(text)
    d = loaders.DenseFile(b)
    assert d.model == "m\u00e9/x" and set(d.tensors) == {'a"b', "t"}
    assert d.tensors['a"b'] == {"offset": 64, "size": 16, "shape": [4, 2], "dtype": "BF16"}
    assert bytes(d.raw('a"b')) == bytes(range(64, 80))
    with pytest.raises(KeyError):
        d.raw("missing")
    d.close()
    for bad in ('{"tensors": {"t": {"offset": 250, "size": 16, "dtype": "U32", "shape": [1]}}}',   # past the end
                '{"tensors": {"t": {"offset": 0, "shape": [1], "dtype": "U32"}}}',                  # no size
                '{"tensors": {"t": {"offset": 0, "size": 4, "dtype": "U32"}',                       # truncated
                '[1, 2]', ''):
        with open(j, "w") as f:
            f.write(bad)
        with pytest.raises(ValueError):
            loaders.DenseFile(b)
    with pytest.raises(ValueError):
        loaders.DenseFile(str(tmp_path / "absent.bin"), j)


def test_quantized_entry_must_be_consistent(tmp_path):
    rng = np.random.default_rng(5)
    t4 = F.synth_affine_tensor(rng, 8, 128, 4)
    W4 = np.ascontiguousarray(t4[1]).view(np.uint32).reshape(8, -1)
    b, j = str(tmp_path / "w.bin"), str(tmp_path / "w.json")
    write_dense(b, j, {"x.weight": ("q", W4, t4[2], t4[3], 4, 64)})
    with open(j) as f:
        man = json.load(f)
    man["tensors"]["x.scales"]["size"] -= 2
    with open(j, "w") as f:
        json.dump(man, f)
    d = loaders.DenseFile(b)
    with pytest.raises(ValueError):
        d.quantized("x.weight")
    del man["tensors"]["x.biases"]
    with open(j, "w") as f:
        json.dump(man, f)
    with pytest.raises(ValueError):
        loaders.DenseFile(b).quantized("x.weight")


def test_gguf_parser_rejects_truncated_and_oversized(tmp_path):
    rng = np.random.default_rng(6)
    g, u, d = F.synth_gguf_layer(rng, 2, 256, 256)
    path = str(tmp_path / "m.gguf")
    write_gguf(path, [("k", 8, "v")], [("blk.0.ffn_gate_exps.weight", 12, [256, 256, 2], g.tobytes()),
                                       ("blk.0.ffn_up_exps.weight", 12, [256, 256, 2], u.tobytes()),
                                       ("blk.0.ffn_down_exps.weight", 14, [256, 256, 2], d.tobytes())])
    whole = open(path, "rb").read()
    gf = loaders.GgufFile(path)
    assert gf.alignment == 32 and gf.expert_geometry(0) == (2, 256, 256, (12, 12, 14))
    with pytest.raises(ValueError):
        gf.expert_geometry(1)
    gf.close()
    for cut in (20, 40, 120, len(whole) - 1):          # header, key/values, tensor infos, data
        with open(path, "wb") as f:
            f.write(whole[:cut])
        with pytest.raises(ValueError):
            loaders.GgufFile(path)
    with open(path, "wb") as f:                        # a tensor count that cannot be true
        f.write(whole[:8] + struct.pack("<Q", 1 << 40) + whole[16:])
    with pytest.raises(ValueError):
        loaders.GgufFile(path)
    # a type the library does not read keeps its directory entry but has no data
    write_gguf(path, [], [("odd", 2, [32], bytes(18))])
    gf = loaders.GgufFile(path)
    assert gf.infos["odd"][0] == 2
    with pytest.raises(ValueError):
        gf.tensor_bytes("odd")
