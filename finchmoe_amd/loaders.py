"""Readers of the reference's weight files, feeding the C ABI.

    ExpertFiles   packed_experts*/layer_XX.bin (finchmoe/repack_experts.py:349-351, 388;
                  finchmoe/infer.m:15421-15425): 256 expert blobs back to back, uploaded verbatim
    DenseFile     model_weights_quant.bin + .json (finchmoe/quantize_non_experts.py:365-386;
                  finchmoe/infer.m:727-786, 859-900): manifest {"tensors": {name: {offset, size,
                  shape, dtype, bits, group_size}}}; a quantized tensor is three entries,
                  NAME.weight (U32), NAME.scales, NAME.biases (BF16)
    GgufFile      GGUF v2/v3 container (finchmoe/infer.m:1025-1247): header, key/values (skipped
                  except general.alignment), tensor infos, aligned data section; the stacked
                  expert tensors blk.N.ffn_{gate,up,down}_exps.weight with dims [in, out, experts]

Files are memory-mapped and handed to the upload calls in place; nothing is converted.
"""
import json
import os
import struct

import numpy as np

GGML_BLOCK = {0: (1, 4), 1: (1, 2), 8: (32, 34), 12: (256, 144), 14: (256, 210), 30: (1, 2)}
"""ggml type -> (elements per block, bytes per block): F32, F16, Q8_0, Q4_K, Q6_K, BF16."""


def _map(path):
    """Read-only byte view of a file; the mapping lives as long as views of it do."""
    if os.path.getsize(path) == 0:
        raise ValueError("%s is empty" % path)
    return np.memmap(path, dtype=np.uint8, mode="r")


class ExpertFiles:
    """layer_%02d.bin files of one packed_experts directory."""

    def __init__(self, directory, n_layers=40, pattern="layer_%02d.bin"):
        self.directory, self.n_layers, self.pattern = directory, n_layers, pattern

    def path(self, layer):
        return os.path.join(self.directory, self.pattern % layer)

    def upload(self, ctx, layers=None):
        """ctx: a FinchHip with experts_config() done.  The file size must be
        n_experts * expert_size exactly (infer.m:15421-15425 reads at e * expert_size)."""
        want = ctx.expert_size() * ctx.n_experts
        for layer in (range(self.n_layers) if layers is None else layers):
            m = _map(self.path(layer))
            if len(m) != want:
                raise ValueError("%s: %d bytes, expected %d" % (self.path(layer), len(m), want))
            ctx.experts_upload_layer(layer, m)


class DenseFile:
    """model_weights_quant.bin with its JSON manifest."""

    def __init__(self, bin_path, json_path=None):
        if json_path is None:
            json_path = os.path.splitext(bin_path)[0] + ".json"
        with open(json_path) as f:
            root = json.load(f)
        if "tensors" not in root:
            raise ValueError("%s: no 'tensors' key" % json_path)      # infer.m:747-750
        self.tensors = root["tensors"]
        self.model = root.get("model")
        self.map = _map(bin_path)
        for name, t in self.tensors.items():
            if t["offset"] + t["size"] > len(self.map):
                raise ValueError("%s: %s ends past the file" % (bin_path, name))

    def close(self):
        self.map = None

    def raw(self, name, dtype=np.uint8):
        """The bytes of one manifest entry (BF16 norm weights: dtype=np.uint16)."""
        t = self.tensors[name]
        return self.map[t["offset"]:t["offset"] + t["size"]].view(dtype)

    def quantized(self, weight_name):
        """(W u32 [out, in*bits/32], S u16, B u16, out_dim, in_dim, bits, group_size) of a
        quantized tensor given its NAME.weight entry."""
        t = self.tensors[weight_name]
        if t["dtype"] != "U32":
            raise ValueError("%s is %s, not a packed tensor" % (weight_name, t["dtype"]))
        bits, gs = int(t["bits"]), int(t["group_size"])
        out_dim, packed_cols = t["shape"]
        in_dim = packed_cols * 32 // bits
        if in_dim % gs:
            raise ValueError("%s: in_dim %d is not a multiple of the group size %d" % (weight_name, in_dim, gs))
        base = weight_name[:-len(".weight")] if weight_name.endswith(".weight") else weight_name
        W = self.raw(weight_name, np.uint32).reshape(out_dim, packed_cols)
        S = self.raw(base + ".scales", np.uint16).reshape(out_dim, in_dim // gs)
        B = self.raw(base + ".biases", np.uint16).reshape(out_dim, in_dim // gs)
        return W, S, B, out_dim, in_dim, bits, gs

    def register(self, ctx, weight_name):
        """-> fm_tensor handle of the tensor, resident on the device."""
        W, S, B, out_dim, in_dim, bits, gs = self.quantized(weight_name)
        return ctx.tensor_register(W, S, B, out_dim, in_dim, bits, gs)


class GgufFile:
    """Tensor directory of a GGUF file; data stays in the mapping."""

    _SCALAR = {0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 6: "f", 7: "?", 10: "Q", 11: "q", 12: "d"}

    def __init__(self, path):
        self.map = _map(path)
        m, self.pos = self.map, 0
        if len(m) < 24 or bytes(m[:4]) != b"GGUF":
            raise ValueError("%s is not a GGUF file" % path)              # infer.m:1041
        self.pos = 4
        self.version = self._u32()
        n_tensors, n_kv = self._u64(), self._u64()
        self.kv = {}
        for _ in range(n_kv):
            key = self._str()
            self.kv[key] = self._value(self._u32())
        self.alignment = int(self.kv.get("general.alignment", 32))
        self.infos = {}
        for _ in range(n_tensors):
            name = self._str()
            nd = self._u32()
            dims = [self._u64() for _ in range(nd)]
            gtype, off = self._u32(), self._u64()
            self.infos[name] = (gtype, dims, off)
        self.data_off = (self.pos + self.alignment - 1) // self.alignment * self.alignment

    def close(self):
        self.map = None

    def _take(self, fmt):
        v = struct.unpack_from("<" + fmt, self.map, self.pos)[0]
        self.pos += struct.calcsize("<" + fmt)
        return v

    def _u32(self):
        return self._take("I")

    def _u64(self):
        return self._take("Q")

    def _str(self):
        n = self._u64()
        if self.pos + n > len(self.map):
            raise ValueError("string runs past the file")
        s = bytes(self.map[self.pos:self.pos + n]).decode("utf-8", "replace")
        self.pos += n
        return s

    def _value(self, vt):
        if vt in self._SCALAR:
            return self._take(self._SCALAR[vt])
        if vt == 8:
            return self._str()
        if vt == 9:
            at, n = self._u32(), self._u64()
            return [self._value(at) for _ in range(n)]
        raise ValueError("unknown GGUF value type %d" % vt)

    def row_bytes(self, name):
        gtype, dims, _ = self.infos[name]
        be, bs = GGML_BLOCK[gtype]
        return dims[0] // be * bs                                         # infer.m:1141-1143

    def tensor_bytes(self, name):
        """(ggml type, dims as stored [in, out, ...], uint8 view of the tensor's bytes)."""
        gtype, dims, off = self.infos[name]
        n = self.row_bytes(name)
        for d in dims[1:]:
            n *= d
        start = self.data_off + off
        if start + n > len(self.map):
            raise ValueError("%s ends past the file" % name)
        return gtype, dims, self.map[start:start + n]

    def expert_layers(self):
        """Layers that have all three stacked expert tensors."""
        out = []
        for name in self.infos:
            if name.startswith("blk.") and name.endswith(".ffn_gate_exps.weight"):
                layer = int(name.split(".")[1])
                if all("blk.%d.ffn_%s_exps.weight" % (layer, k) in self.infos for k in ("up", "down")):
                    out.append(layer)
        return sorted(out)

    def expert_geometry(self, layer=None):
        """(n_experts, hidden, inter, (gate, up, down) ggml types) from the tensor dims
        [in, out, experts] (infer.m:1138-1146)."""
        if layer is None:
            layer = self.expert_layers()[0]
        g = self.infos["blk.%d.ffn_gate_exps.weight" % layer]
        u = self.infos["blk.%d.ffn_up_exps.weight" % layer]
        d = self.infos["blk.%d.ffn_down_exps.weight" % layer]
        hidden, inter, n_experts = g[1][0], g[1][1], g[1][2]
        if d[1][:3] != [inter, hidden, n_experts] or u[1] != g[1]:
            raise ValueError("expert tensors of layer %d disagree on their shapes" % layer)
        return n_experts, hidden, inter, (g[0], u[0], d[0])

    def upload_experts(self, ctx, layers=None):
        """ctx: a FinchHip with gguf_config() done; layer N of the file -> layer N of the store."""
        for layer in (self.expert_layers() if layers is None else layers):
            parts = [self.tensor_bytes("blk.%d.ffn_%s_exps.weight" % (layer, k))[2]
                     for k in ("gate", "up", "down")]
            ctx.gguf_upload_layer(layer, *parts)
