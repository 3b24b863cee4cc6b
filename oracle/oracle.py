"""ctypes/numpy front end of the CPU oracle (libfm_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py.  Nothing under finchmoe_amd/ imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

SCALE_BF16, SCALE_FP16 = 0, 1
Q4_K, Q6_K = 12, 14


class ExpertLayout(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in (
        "gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b",
        "down_w", "down_s", "down_b", "expert_size")]


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "libfm_oracle.so"])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libfm_oracle.so")
        if not os.path.exists(path):
            build()
        L = C.CDLL(path)
        vp, f32p, i32p, u8p, u16p = C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p
        i = C.c_int
        L.orc_bf16_to_f32.restype = C.c_float
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_fp16_to_f32.restype = C.c_float
        L.orc_fp16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_bf16_trunc.restype = C.c_uint16
        L.orc_f32_to_bf16_trunc.argtypes = [C.c_float]
        L.orc_f32_to_fp16_rne.restype = C.c_uint16
        L.orc_f32_to_fp16_rne.argtypes = [C.c_float]
        L.orc_f32_to_bf16_rne.restype = C.c_uint16
        L.orc_f32_to_bf16_rne.argtypes = [C.c_float]
        L.orc_expert_layout_affine.argtypes = [i, i, i, i, C.POINTER(ExpertLayout)]
        L.orc_pack_3bit.argtypes = [u8p, C.c_size_t, u8p]
        L.orc_unpack_3bit.argtypes = [u8p, C.c_size_t, u8p]
        L.orc_pack_u32.argtypes = [u8p, C.c_size_t, i, vp]
        L.orc_unpack_u32.argtypes = [vp, C.c_size_t, i, u8p]
        L.orc_quantize_affine.argtypes = [f32p, i, i, i, i, u8p, u16p, u16p]
        L.orc_dequant_affine.argtypes = [vp, u16p, u16p, i, i, i, i, i, u8p, f32p]
        L.orc_get_scale_min_k4.argtypes = [i, u8p, u8p, u8p]
        L.orc_gguf_dequant_row.argtypes = [vp, f32p, i, i]
        L.orc_gguf_block_value_wordform.restype = C.c_float
        L.orc_gguf_block_value_wordform.argtypes = [u8p, i, i]
        L.orc_gguf_row_bytes.restype = C.c_size_t
        L.orc_gguf_row_bytes.argtypes = [i, i]
        L.orc_dequant_matvec.argtypes = [vp, u16p, u16p, f32p, f32p, i, i, i, i, i]
        L.orc_dequant_matvec_mt.argtypes = [vp, u16p, u16p, f32p, f32p, i, i, i, i, i, i]
        L.orc_dequant_matvec_bf16model.argtypes = [vp, u16p, u16p, f32p, f32p, i, i, i, i, i]
        L.orc_swiglu.argtypes = [f32p, f32p, f32p, i]
        L.orc_softmax.argtypes = [f32p, i]
        L.orc_topk.argtypes = [f32p, i, i, i32p, f32p]
        L.orc_normalize_weights.argtypes = [f32p, i]
        L.orc_vec_madd.argtypes = [f32p, f32p, C.c_float, i]
        L.orc_moe_experts_forward.argtypes = [u8p, i, i, i, i, i, f32p, i32p, f32p, i, i,
                                              f32p, f32p, f32p, f32p, f32p, i]
        L.orc_moe_gguf_forward.argtypes = [u8p, u8p, u8p, i, i, i, i, i, f32p, i32p, f32p,
                                           i, i, f32p, f32p, i]
        L.orc_rms_norm.argtypes = [f32p, u16p, f32p, i, C.c_float]
        L.orc_layer_tail.argtypes = [vp, u16p, u16p, i, i, i, i, i, f32p, f32p, f32p, i, f32p, f32p,
                                     u16p, C.c_float, f32p, f32p]
        _LIB = L
    return _LIB


_REF = None


def ref_lib():
    """oracle/_ref/libfm_ref.so: the reference's own CPU functions (finchmoe/infer.m:686-702,
    1575-1881) compiled by build_ref.sh.  None when it has not been built (the reference tree
    is not mounted and no prebuilt copy travelled with the tree)."""
    global _REF
    if _REF is None:
        path = os.path.join(_HERE, "_ref", "libfm_ref.so")
        if not os.path.exists(path):
            return None
        R = C.CDLL(path)
        vp, i, f = C.c_void_p, C.c_int, C.c_float
        R.ref_bf16_to_f32.restype = f
        R.ref_bf16_to_f32.argtypes = [C.c_uint16]
        R.ref_f32_to_bf16.restype = C.c_uint16
        R.ref_f32_to_bf16.argtypes = [f]
        R.ref_fp16_to_f32.restype = f
        R.ref_fp16_to_f32.argtypes = [C.c_uint16]
        R.ref_get_scale_min_k4.argtypes = [i, vp, vp, vp]
        R.ref_gguf_dequant_row.argtypes = [vp, vp, i, i]
        R.ref_cpu_dequant_matvec.argtypes = [vp, vp, vp, vp, vp, i, i, i, i]
        R.ref_cpu_rms_norm.argtypes = [vp, vp, vp, i, f]
        R.ref_cpu_swiglu.argtypes = [vp, vp, vp, i]
        R.ref_cpu_sigmoid.restype = f
        R.ref_cpu_sigmoid.argtypes = [f]
        R.ref_cpu_softmax.argtypes = [vp, i]
        R.ref_cpu_topk.argtypes = [vp, i, i, vp, vp]
        R.ref_cpu_normalize_weights.argtypes = [vp, i]
        R.ref_cpu_vec_madd.argtypes = [vp, vp, f, i]
        _REF = R
    return _REF


def _p(a):
    return None if a is None else a.ctypes.data


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


# ---------------------------------------------------------------- scalars
def bf16_to_f32(u16):
    u16 = _c(u16, np.uint16)
    return (u16.astype(np.uint32) << 16).view(np.float32)


def fp16_to_f32_scalar(h):
    return lib().orc_fp16_to_f32(int(h))


def expert_layout(hidden, inter, group_size, bits):
    lo = ExpertLayout()
    lib().orc_expert_layout_affine(hidden, inter, group_size, bits, C.byref(lo))
    return lo


# ---------------------------------------------------------------- packers
def pack_3bit(codes):
    codes = _c(codes, np.uint8).reshape(-1)
    out = np.empty(codes.size * 3 // 8, np.uint8)
    lib().orc_pack_3bit(_p(codes), codes.size, _p(out))
    return out


def unpack_3bit(packed, n):
    packed = _c(packed, np.uint8).reshape(-1)
    out = np.empty(n, np.uint8)
    lib().orc_unpack_3bit(_p(packed), n, _p(out))
    return out


def pack_u32(codes, bits):
    codes = _c(codes, np.uint8).reshape(-1)
    out = np.empty(codes.size * bits // 32, np.uint32)
    lib().orc_pack_u32(_p(codes), codes.size, bits, _p(out))
    return out


def unpack_u32(packed, n, bits):
    packed = _c(packed, np.uint32).reshape(-1)
    out = np.empty(n, np.uint8)
    lib().orc_unpack_u32(_p(packed), n, bits, _p(out))
    return out


def quantize_affine(w, bits, group_size=64):
    w = _c(w, np.float32)
    od, idim = w.shape
    codes = np.empty((od, idim), np.uint8)
    s = np.empty((od, idim // group_size), np.uint16)
    b = np.empty_like(s)
    lib().orc_quantize_affine(_p(w), od, idim, group_size, bits, _p(codes), _p(s), _p(b))
    return codes, s, b


# ---------------------------------------------------------------- dequant
def dequant_affine(W, S, B, out_dim, in_dim, bits, group_size=64, scale_dtype=SCALE_BF16):
    W = np.ascontiguousarray(W)
    S = _c(S, np.uint16)
    B = _c(B, np.uint16)
    codes = np.empty((out_dim, in_dim), np.uint8)
    w = np.empty((out_dim, in_dim), np.float32)
    lib().orc_dequant_affine(_p(W), _p(S), _p(B), out_dim, in_dim, group_size, bits,
                             scale_dtype, _p(codes), _p(w))
    return codes, w


def f32_to_fp16_rne(a):
    a = _c(a, np.float32)
    L = lib()
    flat = a.reshape(-1)
    out = np.empty(flat.size, np.uint16)
    for k in range(flat.size):
        out[k] = L.orc_f32_to_fp16_rne(float(flat[k]))
    return out.reshape(a.shape)


def gguf_row_bytes(in_dim, ggml_type):
    return lib().orc_gguf_row_bytes(in_dim, ggml_type)


def gguf_dequant(W, out_dim, in_dim, ggml_type):
    W = _c(W, np.uint8).reshape(-1)
    rb = gguf_row_bytes(in_dim, ggml_type)
    y = np.empty((out_dim, in_dim), np.float32)
    L = lib()
    for r in range(out_dim):
        L.orc_gguf_dequant_row(W.ctypes.data + r * rb, y[r].ctypes.data, in_dim, ggml_type)
    return y


def gguf_block_value_wordform(block, e, ggml_type):
    block = _c(block, np.uint8)
    return lib().orc_gguf_block_value_wordform(_p(block), e, ggml_type)


# ---------------------------------------------------------------- matvec
def dequant_matvec(W, S, B, x, out_dim, in_dim, bits, group_size=64,
                   scale_dtype=SCALE_BF16, nthreads=1):
    W = np.ascontiguousarray(W)
    S = None if S is None else _c(S, np.uint16)
    B = None if B is None else _c(B, np.uint16)
    x = _c(x, np.float32)
    out = np.empty(out_dim, np.float32)
    lib().orc_dequant_matvec_mt(_p(W), _p(S), _p(B), _p(x), _p(out), out_dim, in_dim,
                                group_size, bits, scale_dtype, nthreads)
    return out


def dequant_matvec_bf16model(W, S, B, x, out_dim, in_dim, bits, group_size=64,
                             scale_dtype=SCALE_BF16):
    W = np.ascontiguousarray(W)
    S = _c(S, np.uint16)
    B = _c(B, np.uint16)
    x = _c(x, np.float32)
    out = np.empty(out_dim, np.float32)
    lib().orc_dequant_matvec_bf16model(_p(W), _p(S), _p(B), _p(x), _p(out), out_dim, in_dim,
                                       group_size, bits, scale_dtype)
    return out


def swiglu(g, u):
    g = _c(g, np.float32)
    u = _c(u, np.float32)
    out = np.empty_like(g)
    lib().orc_swiglu(_p(g), _p(u), _p(out), g.size)
    return out


def rms_norm(x, w_bf16, eps=1e-6):
    x = _c(x, np.float32)
    w = _c(w_bf16, np.uint16)
    out = np.empty_like(x)
    lib().orc_rms_norm(_p(x), _p(w), _p(out), x.size, eps)
    return out


def layer_tail(sdW, sdS, sdB, h_mid, expert_out, params, K, shared_gate, shared_up, next_norm_w,
               bits=4, group_size=64, scale_dtype=SCALE_BF16, eps=1e-6):
    """-> (hidden_out, next_in or None)"""
    sdW = np.ascontiguousarray(sdW)
    sdS, sdB = _c(sdS, np.uint16), _c(sdB, np.uint16)
    h_mid = _c(h_mid, np.float32)
    eo = _c(expert_out, np.float32)
    params = _c(params, np.float32)
    sg, su = _c(shared_gate, np.float32), _c(shared_up, np.float32)
    nw = None if next_norm_w is None else _c(next_norm_w, np.uint16)
    hidden, si = h_mid.size, sg.size
    hid = np.empty(hidden, np.float32)
    nxt = None if nw is None else np.empty(hidden, np.float32)
    lib().orc_layer_tail(_p(sdW), _p(sdS), _p(sdB), hidden, si, group_size, bits, scale_dtype,
                         _p(h_mid), _p(eo), _p(params), K, _p(sg), _p(su), _p(nw), eps,
                         _p(hid), _p(nxt))
    return hid, nxt


def softmax(x):
    x = _c(x, np.float32).copy()
    lib().orc_softmax(_p(x), x.size)
    return x


def topk(scores, K):
    scores = _c(scores, np.float32)
    idx = np.empty(K, np.int32)
    val = np.empty(K, np.float32)
    lib().orc_topk(_p(scores), scores.size, K, _p(idx), _p(val))
    return idx, val


def normalize_weights(w):
    w = _c(w, np.float32).copy()
    lib().orc_normalize_weights(_p(w), w.size)
    return w


def route(logits, K):
    """softmax -> top-K -> renormalise, the reference's CPU routing
    (infer.m:9285-9289)."""
    p = softmax(logits)
    idx, val = topk(p, K)
    return idx, normalize_weights(val)


# ---------------------------------------------------------------- expert block
def moe_experts_forward(layer_blob, x, idx, w, hidden=2048, inter=512, bits=3,
                        group_size=64, scale_dtype=SCALE_BF16, guard=0, nthreads=1,
                        stages=False):
    layer_blob = _c(layer_blob, np.uint8).reshape(-1)
    x = _c(x, np.float32)
    idx = _c(idx, np.int32)
    w = _c(w, np.float32)
    K = idx.size
    moe = np.zeros(hidden, np.float32)
    eo = np.empty((K, hidden), np.float32)
    g = np.empty((K, inter), np.float32) if stages else None
    u = np.empty((K, inter), np.float32) if stages else None
    a = np.empty((K, inter), np.float32) if stages else None
    lib().orc_moe_experts_forward(_p(layer_blob), hidden, inter, group_size, bits,
                                  scale_dtype, _p(x), _p(idx), _p(w), K, guard,
                                  _p(moe), _p(eo), _p(g), _p(u), _p(a), nthreads)
    if stages:
        return moe, eo, g, u, a
    return moe, eo


def moe_gguf_forward(gate, up, down, x, idx, w, hidden=2048, inter=512,
                     types=(Q4_K, Q4_K, Q6_K), guard=0, nthreads=1):
    gate = _c(gate, np.uint8).reshape(-1)
    up = _c(up, np.uint8).reshape(-1)
    down = _c(down, np.uint8).reshape(-1)
    x = _c(x, np.float32)
    idx = _c(idx, np.int32)
    w = _c(w, np.float32)
    K = idx.size
    moe = np.zeros(hidden, np.float32)
    eo = np.empty((K, hidden), np.float32)
    lib().orc_moe_gguf_forward(_p(gate), _p(up), _p(down), types[0], types[1], types[2],
                               hidden, inter, _p(x), _p(idx), _p(w), K, guard,
                               _p(moe), _p(eo), nthreads)
    return moe, eo
