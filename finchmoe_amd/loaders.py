"""Python face of the C readers of the reference's weight files and of its quantizer
(finchmoe_amd/host/finch_files.c in libfinchops.so); parsing, mapping and quantising happen there.

    quantize_affine_pack   finchmoe/repack_experts.py:232-333, finchmoe/quantize_model.py:13-47,
                           finchmoe/quantize_non_experts.py:30-69
    ExpertFiles   packed_experts*/layer_XX.bin (finchmoe/repack_experts.py:349-351, 388;
                  finchmoe/infer.m:15421-15425): 256 expert blobs back to back, uploaded verbatim
    DenseFile     model_weights_quant.bin + .json (finchmoe/quantize_non_experts.py:365-386;
                  finchmoe/infer.m:727-786, 859-900): manifest {"tensors": {name: {offset, size,
                  shape, dtype, bits, group_size}}}; a quantized tensor is three entries,
                  NAME.weight (U32), NAME.scales, NAME.biases (BF16)
    GgufFile      GGUF v2/v3 container (finchmoe/infer.m:1025-1247): header, key/values (skipped
                  except general.alignment, as the reference does), tensor infos, aligned data
                  section; the stacked expert tensors blk.N.ffn_{gate,up,down}_exps.weight with
                  dims [in, out, experts]

Files are memory-mapped by the C side and handed to the upload calls in place; nothing is
converted.  The upload methods take a FinchHip context; a C caller uses finch_ops_load_expert_dir,
finch_ops_load_dense_tensor and finch_ops_load_gguf_experts instead.
"""
import ctypes as C
import os

import numpy as np

from . import binding

GGML_BLOCK = {0: (1, 4), 1: (1, 2), 8: (32, 34), 12: (256, 144), 14: (256, 210), 30: (1, 2)}
"""ggml type -> (elements per block, bytes per block): F32, F16, Q8_0, Q4_K, Q6_K, BF16."""


class _DenseEntry(C.Structure):      # finch_dense_entry
    _fields_ = [("name", C.c_char_p), ("data", C.c_void_p), ("offset", C.c_uint64), ("size", C.c_size_t),
                ("ndim", C.c_int), ("shape", C.c_int64 * 4), ("dtype", C.c_char * 8), ("bits", C.c_int),
                ("group_size", C.c_int)]


class _GgufTensor(C.Structure):      # finch_gguf_tensor
    _fields_ = [("name", C.c_char_p), ("type", C.c_int), ("ndim", C.c_int), ("dims", C.c_uint64 * 4),
                ("data", C.c_void_p), ("nbytes", C.c_size_t)]


_L = None


def lib():
    """libfinchops.so with the file functions typed."""
    global _L
    if _L is not None:
        return _L
    binding.load()       # libfinchops.so links against libfinchhip.so; load that one first
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libfinchops.so")
    if not os.path.exists(path):
        raise OSError("%s is not built (run finchmoe_amd/build.py)" % path)
    L = C.CDLL(path)
    vp, i, sz, s = C.c_void_p, C.c_int, C.c_size_t, C.c_char_p
    pi = C.POINTER(C.c_int)
    L.finch_files_last_error.restype = s
    L.finch_quantize_affine_pack.argtypes = [vp, i, i, i, i, vp, vp, vp]
    L.finch_expert_blob_size.argtypes = [i, i, i, i]
    L.finch_expert_blob_size.restype = sz
    L.finch_quantize_expert.argtypes = [vp, vp, vp, i, i, i, i, vp]
    L.finch_file_map.argtypes = [s, C.POINTER(vp), C.POINTER(sz)]
    L.finch_file_unmap.argtypes = [vp, sz]
    L.finch_file_unmap.restype = None
    L.finch_expert_layer_path.argtypes = [s, i, C.c_char_p, sz]
    L.finch_ops_load_expert_dir.argtypes = [s, i]
    L.finch_ops_open_dense.argtypes = [s, s]
    L.finch_ops_open_dense.restype = vp
    L.finch_ops_close_dense.argtypes = [vp]
    L.finch_ops_close_dense.restype = None
    L.finch_dense_count.argtypes = [vp]
    L.finch_dense_model.argtypes = [vp]
    L.finch_dense_model.restype = s
    L.finch_dense_entry_at.argtypes = [vp, i, C.POINTER(_DenseEntry)]
    L.finch_dense_find.argtypes = [vp, s, C.POINTER(_DenseEntry)]
    L.finch_dense_quantized.argtypes = [vp, s, C.POINTER(vp), C.POINTER(vp), C.POINTER(vp), pi, pi, pi, pi]
    L.finch_ops_load_dense_tensor.argtypes = [vp, s]
    L.finch_ops_open_gguf.argtypes = [s]
    L.finch_ops_open_gguf.restype = vp
    L.finch_ops_close_gguf.argtypes = [vp]
    L.finch_ops_close_gguf.restype = None
    for f in (L.finch_gguf_version, L.finch_gguf_alignment, L.finch_gguf_count):
        f.argtypes = [vp]
    L.finch_gguf_data_offset.argtypes = [vp]
    L.finch_gguf_data_offset.restype = C.c_uint64
    L.finch_gguf_tensor_at.argtypes = [vp, i, C.POINTER(_GgufTensor)]
    L.finch_gguf_find.argtypes = [vp, s, C.POINTER(_GgufTensor)]
    L.finch_ggml_block.argtypes = [i, pi, pi]
    L.finch_gguf_expert_geometry.argtypes = [vp, i, pi, pi, pi, C.c_int * 3]
    L.finch_gguf_has_expert_layer.argtypes = [vp, i]
    L.finch_ops_load_gguf_experts.argtypes = [vp, i]
    _L = L
    return L


def _err():
    return lib().finch_files_last_error().decode("utf-8", "replace")


def _view(owner, addr, nbytes):
    """Read-only uint8 view of C memory that keeps `owner` (the mapping's holder) alive."""
    if not nbytes:
        return np.empty(0, np.uint8)
    buf = (C.c_uint8 * nbytes).from_address(addr)
    buf._owner = owner
    a = np.ctypeslib.as_array(buf)
    a.flags.writeable = False
    return a


def quantize_affine_pack(w, bits, group_size=64):
    """w [out_dim][in_dim] fp32 -> (packed uint8 [out_dim][in_dim*bits/8], scales u16, biases u16
    [out_dim][in_dim/group_size]), bit for bit what the reference's quantizers write."""
    w = np.ascontiguousarray(w, np.float32)
    if w.ndim != 2:
        raise ValueError("w must be 2-D")
    out_dim, in_dim = w.shape
    packed = np.empty((out_dim, in_dim * bits // 8), np.uint8)
    S = np.empty((out_dim, max(in_dim // group_size, 1)), np.uint16)
    B = np.empty_like(S)
    rc = lib().finch_quantize_affine_pack(w.ctypes.data, out_dim, in_dim, group_size, bits,
                                          packed.ctypes.data, S.ctypes.data, B.ctypes.data)
    if rc:
        raise ValueError(_err())
    return packed, S, B


def quantize_expert(gate, up, down, bits, group_size=64):
    """Three fp32 matrices of one expert -> its blob in the layer-file layout (uint8)."""
    gate, up, down = (np.ascontiguousarray(a, np.float32) for a in (gate, up, down))
    inter, hidden = gate.shape
    if up.shape != (inter, hidden) or down.shape != (hidden, inter):
        raise ValueError("gate/up must be [inter][hidden], down [hidden][inter]")
    n = lib().finch_expert_blob_size(hidden, inter, group_size, bits)
    if not n:
        raise ValueError("expert geometry %dx%d, group %d, %d bits is not representable" % (hidden, inter, group_size, bits))
    blob = np.empty(n, np.uint8)
    rc = lib().finch_quantize_expert(gate.ctypes.data, up.ctypes.data, down.ctypes.data, hidden, inter,
                                     group_size, bits, blob.ctypes.data)
    if rc:
        raise ValueError(_err())
    return blob


class _Mapping:
    """One file mapped by finch_file_map, unmapped when the last view of it goes."""

    def __init__(self, path):
        p, n = C.c_void_p(), C.c_size_t()
        if lib().finch_file_map(path.encode(), C.byref(p), C.byref(n)):
            raise ValueError(_err())
        self.addr, self.nbytes = p.value, n.value

    def view(self):
        return _view(self, self.addr, self.nbytes)

    def __del__(self):
        if getattr(self, "addr", None):
            lib().finch_file_unmap(self.addr, self.nbytes)
            self.addr = None


class ExpertFiles:
    """layer_%02d.bin files of one packed_experts directory."""

    def __init__(self, directory, n_layers=40):
        self.directory, self.n_layers = directory, n_layers

    def path(self, layer):
        buf = C.create_string_buffer(1024)
        if lib().finch_expert_layer_path(self.directory.encode(), layer, buf, len(buf)):
            raise ValueError(_err())
        return buf.value.decode()

    def upload(self, ctx, layers=None):
        """ctx: a FinchHip with experts_config() done.  The file size must be
        n_experts * expert_size exactly (infer.m:15421-15425 reads at e * expert_size)."""
        want = ctx.expert_size() * ctx.n_experts
        for layer in (range(self.n_layers) if layers is None else layers):
            m = _Mapping(self.path(layer))
            if m.nbytes != want:
                raise ValueError("%s: %d bytes, expected %d" % (self.path(layer), m.nbytes, want))
            ctx.experts_upload_layer(layer, m.view())


class DenseFile:
    """model_weights_quant.bin with its JSON manifest."""

    def __init__(self, bin_path, json_path=None):
        self.h = lib().finch_ops_open_dense(bin_path.encode(), json_path.encode() if json_path else None)
        if not self.h:
            raise ValueError(_err())
        m = lib().finch_dense_model(self.h)
        self.model = m.decode() if m is not None else None
        self.tensors = {}
        e = _DenseEntry()
        for i in range(lib().finch_dense_count(self.h)):
            lib().finch_dense_entry_at(self.h, i, C.byref(e))
            t = {"offset": e.offset, "size": e.size, "shape": list(e.shape[:e.ndim]), "dtype": e.dtype.decode()}
            if e.bits:
                t["bits"], t["group_size"] = e.bits, e.group_size
            self.tensors[e.name.decode()] = t

    def close(self):
        """Unmaps the file: views handed out before are dead after this."""
        if self.h:
            lib().finch_ops_close_dense(self.h)
            self.h = None

    __del__ = close

    def raw(self, name, dtype=np.uint8):
        """The bytes of one manifest entry (BF16 norm weights: dtype=np.uint16)."""
        e = _DenseEntry()
        if lib().finch_dense_find(self.h, name.encode(), C.byref(e)):
            raise KeyError(_err())
        return _view(self, e.data, e.size).view(dtype)

    def quantized(self, weight_name):
        """(W u32 [out, in*bits/32], S u16, B u16, out_dim, in_dim, bits, group_size) of a
        quantized tensor given its NAME.weight entry."""
        W, S, B = C.c_void_p(), C.c_void_p(), C.c_void_p()
        od, idim, bits, gs = C.c_int(), C.c_int(), C.c_int(), C.c_int()
        if lib().finch_dense_quantized(self.h, weight_name.encode(), C.byref(W), C.byref(S), C.byref(B),
                                       C.byref(od), C.byref(idim), C.byref(bits), C.byref(gs)):
            raise ValueError(_err())
        od, idim, bits, gs = od.value, idim.value, bits.value, gs.value
        cols, ng = idim * bits // 32, idim // gs
        Wv = _view(self, W.value, od * cols * 4).view(np.uint32).reshape(od, cols)
        Sv = _view(self, S.value, od * ng * 2).view(np.uint16).reshape(od, ng)
        Bv = _view(self, B.value, od * ng * 2).view(np.uint16).reshape(od, ng)
        return Wv, Sv, Bv, od, idim, bits, gs

    def register(self, ctx, weight_name):
        """-> fm_tensor handle of the tensor, resident on the device."""
        W, S, B, out_dim, in_dim, bits, gs = self.quantized(weight_name)
        return ctx.tensor_register(W, S, B, out_dim, in_dim, bits, gs)


class GgufFile:
    """Tensor directory of a GGUF file; data stays in the mapping."""

    def __init__(self, path):
        self.h = lib().finch_ops_open_gguf(path.encode())
        if not self.h:
            raise ValueError(_err())
        L = lib()
        self.version, self.alignment = L.finch_gguf_version(self.h), L.finch_gguf_alignment(self.h)
        self.data_off = L.finch_gguf_data_offset(self.h)
        self.infos = {}
        t = _GgufTensor()
        for i in range(L.finch_gguf_count(self.h)):
            L.finch_gguf_tensor_at(self.h, i, C.byref(t))
            self.infos[t.name.decode()] = (t.type, list(t.dims[:t.ndim]), t.nbytes)

    def close(self):
        """Unmaps the file: views handed out before are dead after this."""
        if self.h:
            lib().finch_ops_close_gguf(self.h)
            self.h = None

    __del__ = close

    def row_bytes(self, name):
        gtype, dims, _ = self.infos[name]
        be, bs = C.c_int(), C.c_int()
        if not lib().finch_ggml_block(gtype, C.byref(be), C.byref(bs)):
            raise ValueError("ggml type %d is not read by this library" % gtype)
        return dims[0] // be.value * bs.value                             # infer.m:1141-1143

    def tensor_bytes(self, name):
        """(ggml type, dims as stored [in, out, ...], uint8 view of the tensor's bytes)."""
        t = _GgufTensor()
        if lib().finch_gguf_find(self.h, name.encode(), C.byref(t)):
            raise KeyError(_err())
        if not t.data:
            raise ValueError("%s: ggml type %d is not read by this library" % (name, t.type))
        return t.type, list(t.dims[:t.ndim]), _view(self, t.data, t.nbytes)

    def expert_layers(self):
        """Layers that have all three stacked expert tensors."""
        cand = {int(n.split(".")[1]) for n in self.infos
                if n.startswith("blk.") and n.endswith(".ffn_gate_exps.weight")}
        return sorted(l for l in cand if lib().finch_gguf_has_expert_layer(self.h, l))

    def expert_geometry(self, layer=None):
        """(n_experts, hidden, inter, (gate, up, down) ggml types) from the tensor dims
        [in, out, experts] (infer.m:1138-1146)."""
        ne, hh, ii, types = C.c_int(), C.c_int(), C.c_int(), (C.c_int * 3)()
        if lib().finch_gguf_expert_geometry(self.h, -1 if layer is None else layer, C.byref(ne),
                                            C.byref(hh), C.byref(ii), types):
            raise ValueError(_err())
        return ne.value, hh.value, ii.value, tuple(types)

    def upload_experts(self, ctx, layers=None):
        """ctx: a FinchHip with gguf_config() done; layer N of the file -> layer N of the store."""
        for layer in (self.expert_layers() if layers is None else layers):
            parts = [self.tensor_bytes("blk.%d.ffn_%s_exps.weight" % (layer, k))[2]
                     for k in ("gate", "up", "down")]
            ctx.gguf_upload_layer(layer, *parts)
