"""ctypes binding of libfinchhip.so (the C ABI of include/finch_hip.h).

Thin by design: pointers and sizes go straight through.  Host entry points take
numpy arrays; *_dev entry points take integer device addresses (for instance
torch.Tensor.data_ptr()).  If the library is missing the import of this module
still succeeds (CPU-only tooling), but creating a context raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

OK, ERR_ARG, ERR_HIP, ERR_STATE, ERR_UNSUPPORTED, ERR_NOMEM = 0, -1, -2, -3, -4, -5
FORM_PLAIN_DENSE, FORM_PLAIN_GGUF, FORM_NO_DENSE_GEMM, FORM_NO_GGUF_GROUP, FORM_GGUF_PHASES = 1, 2, 4, 8, 16
FORM_GGUF_ONE_LAUNCH = 32
SCALE_BF16, SCALE_FP16 = 0, 1
Q4_K, Q6_K = 12, 14
ACCUMULATE, GUARD = 1, 2
GATE, UP, DOWN = 0, 1, 2


class FinchError(RuntimeError):
    def __init__(self, status, msg):
        super().__init__("finch_hip status %d: %s" % (status, msg))
        self.status = status


def lib_path():
    """In-tree library; FINCH_HIP_LIB overrides the path (alternative builds)."""
    return os.environ.get("FINCH_HIP_LIB") or os.path.join(_HERE, "libfinchhip.so")


_LIB = None


def load():
    """Load libfinchhip.so; raises if it has not been built (no fallback)."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = lib_path()
    if not os.path.exists(path):
        raise FinchError(ERR_STATE, "libfinchhip.so not built: run python -m finchmoe_amd.build")
    # One HIP runtime per process.  PyTorch ships its own libamdhip64 (same SONAME as the
    # system one); if it is loaded first, this library's libamdhip64.so.7 dependency binds to
    # it.  Loaded in the other order the process ends up with two runtimes and the second one
    # finds no device.  So when torch is installed, load it first.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(path)
    vp, i, sz = C.c_void_p, C.c_int, C.c_size_t
    sig = {
        "fm_ctx_create": (i, [i, C.POINTER(vp)]),
        "fm_ctx_destroy": (i, [vp]),
        "fm_sync": (i, [vp]),
        "fm_stream": (vp, [vp]),
        "fm_last_error": (C.c_char_p, [vp]),
        "fm_status_string": (C.c_char_p, [i]),
        "fm_timer_start": (i, [vp]),
        "fm_timer_stop": (i, [vp, C.POINTER(C.c_float)]),
        "fm_kernel_timing": (i, [vp, i]),
        "fm_set_wait_limit": (i, [vp, C.c_uint]),
        "fm_set_kernel_forms": (i, [C.c_uint]),
        "fm_reserve": (i, [vp, i, i, C.c_size_t]),
        "fm_release_graphs": (i, [vp]),
        "fm_kernel_timing_read": (i, [vp, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(i)]),
        "fm_stream_probe_dev": (i, [vp, vp, sz, i]),
        "fm_experts_config": (i, [vp, i, i, i, i, i, i, i]),
        "fm_experts_expert_size": (sz, [vp]),
        "fm_experts_upload_layer": (i, [vp, i, vp, sz]),
        "fm_experts_adopt_layer": (i, [vp, i, vp, sz]),
        "fm_moe_decode_dev": (i, [vp, i, vp, vp, vp, i, vp, vp, i]),
        "fm_moe_decode": (i, [vp, i, vp, vp, vp, i, vp, vp, i]),
        "fm_moe_decode_step_dev": (i, [vp, i, i, vp, vp, vp, i, vp, vp, i]),
        "fm_moe_decode_step_noalloc_dev": (i, [vp, i, i, vp, vp, vp, i, vp, i]),
        "fm_moe_prefill_dev": (i, [vp, i, vp, vp, vp, i, i, vp, i]),
        "fm_moe_prefill": (i, [vp, i, vp, vp, vp, i, i, vp, i]),
        "fm_moe_prefill_bf16_dev": (i, [vp, i, vp, vp, vp, i, i, vp, i]),
        "fm_moe_prefill_bf16": (i, [vp, i, vp, vp, vp, i, i, vp, i]),
        "fm_tensor_register": (i, [vp, vp, vp, vp, i, i, i, i, i, C.POINTER(i)]),
        "fm_tensor_adopt": (i, [vp, vp, vp, vp, i, i, i, i, i, C.POINTER(i)]),
        "fm_tensor_release": (i, [vp, i]),
        "fm_matvec_batch_dev": (i, [vp, C.POINTER(i), i, vp, C.POINTER(vp)]),
        "fm_matvec_batch": (i, [vp, C.POINTER(i), i, vp, C.POINTER(vp)]),
        "fm_matvec_prefill_dev": (i, [vp, i, vp, vp, i]),
        "fm_matvec_prefill": (i, [vp, i, vp, vp, i]),
        "fm_route_topk_dev": (i, [vp, vp, i, i, vp, vp, vp, vp]),
        "fm_matvec_batch_route_dev": (i, [vp, C.POINTER(i), i, vp, C.POINTER(vp), i, vp, vp, vp, vp]),
        "fm_layer_tail_dev": (i, [vp, i, vp, vp, vp, i, vp, vp, vp, C.c_float, vp, vp]),
        "fm_moe_decode_tail_dev": (i, [vp, i, vp, vp, vp, i, i, vp, vp, vp, vp, vp, C.c_float, vp, vp]),
        "fm_moe_layer_dev": (i, [vp, i, C.POINTER(i), vp, i, i, vp, vp, C.c_float, vp, vp, vp, vp, vp, vp, vp, vp, vp]),
        "fm_gguf_config": (i, [vp, i, i, i, i, i, i, i]),
        "fm_gguf_upload_layer": (i, [vp, i, vp, sz, vp, sz, vp, sz]),
        "fm_gguf_adopt_layer": (i, [vp, i, vp, sz, vp, sz, vp, sz]),
        "fm_gguf_moe_decode_dev": (i, [vp, i, vp, vp, vp, i, vp, vp, i]),
        "fm_gguf_moe_decode": (i, [vp, i, vp, vp, vp, i, vp, vp, i]),
        "fm_gguf_moe_decode_step_dev": (i, [vp, i, i, vp, vp, vp, i, vp, vp, i]),
        "fm_gguf_moe_prefill_dev": (i, [vp, i, vp, vp, vp, i, i, vp, i]),
        "fm_gguf_moe_prefill": (i, [vp, i, vp, vp, vp, i, i, vp, i]),
        "fm_gguf_matvec": (i, [vp, vp, i, vp, vp, i, i]),
        "fm_dequant_expert": (i, [vp, i, i, i, vp, vp, vp]),
        "fm_dequant_tensor": (i, [vp, i, vp, vp, vp]),
        "fm_gguf_dequant_expert": (i, [vp, i, i, i, vp]),
        "fm_embed_lookup_dev": (i, [vp, i, vp, i, vp]),
        "fm_matvec_prefill_batch_dev": (i, [vp, vp, i, vp, vp, i]),
        "fm_embed_lookup": (i, [vp, i, i, vp]),
    }
    for name, (res, args) in sig.items():
        f = getattr(L, name)
        f.restype = res
        f.argtypes = args
    L._signatures = sig
    _LIB = L
    return L


def _np(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def _ptr(a):
    return None if a is None else a.ctypes.data


class FinchHip:
    """One context = one device + one stream (see include/finch_hip.h)."""

    def __init__(self, device=0):
        self.L = load()
        h = C.c_void_p()
        rc = self.L.fm_ctx_create(device, C.byref(h))
        if rc:
            raise FinchError(rc, "fm_ctx_create failed (no GPU? there is no CPU fallback)")
        self.h = h
        self.hidden = self.inter = None

    def close(self):
        if getattr(self, "h", None):
            self.L.fm_ctx_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _chk(self, rc):
        if rc:
            raise FinchError(rc, self.L.fm_last_error(self.h).decode())

    # ---- misc
    def sync(self):
        self._chk(self.L.fm_sync(self.h))

    def stream(self):
        return self.L.fm_stream(self.h)

    def timer_start(self):
        self._chk(self.L.fm_timer_start(self.h))

    def timer_stop(self):
        ms = C.c_float()
        self._chk(self.L.fm_timer_stop(self.h, C.byref(ms)))
        return ms.value

    def kernel_timing(self, enable):
        self._chk(self.L.fm_kernel_timing(self.h, int(enable)))

    def set_wait_limit(self, polls):
        self._chk(self.L.fm_set_wait_limit(self.h, C.c_uint(polls)))

    def set_kernel_forms(self, forms):
        """Process-wide override of the kernel choice (FORM_* flags; 0 = default)."""
        self._chk(self.L.fm_set_kernel_forms(C.c_uint(forms)))

    def reserve(self, n_groups=0, M=0, workspace_bytes=0):
        """Scratch for steps of n_groups layers / chunks of M positions, before capturing."""
        self._chk(self.L.fm_reserve(self.h, n_groups, M, workspace_bytes))

    def release_graphs(self):
        self._chk(self.L.fm_release_graphs(self.h))

    def kernel_timing_read(self):
        a, b, n = C.c_double(), C.c_double(), C.c_int()
        self._chk(self.L.fm_kernel_timing_read(self.h, C.byref(a), C.byref(b), C.byref(n)))
        return a.value, b.value, n.value

    def stream_probe_dev(self, d_buf, nbytes, pattern=0):
        self._chk(self.L.fm_stream_probe_dev(self.h, d_buf, nbytes, pattern))

    # ---- affine expert store
    def experts_config(self, n_layers, n_experts, hidden=2048, inter=512, group_size=64, bits=3,
                       scale_dtype=SCALE_BF16):
        self._chk(self.L.fm_experts_config(self.h, n_layers, n_experts, hidden, inter, group_size,
                                           bits, scale_dtype))
        self.hidden, self.inter, self.n_experts = hidden, inter, n_experts

    def expert_size(self):
        return self.L.fm_experts_expert_size(self.h)

    def experts_upload_layer(self, layer, blob):
        blob = _np(blob, np.uint8).reshape(-1)
        self._chk(self.L.fm_experts_upload_layer(self.h, layer, _ptr(blob), blob.size))

    def experts_adopt_layer(self, layer, dev_ptr, nbytes):
        self._chk(self.L.fm_experts_adopt_layer(self.h, layer, dev_ptr, nbytes))

    # ---- decode
    def moe_decode(self, layer, x, idx, w, flags=0, out=None, want_expert_out=True):
        x, idx, w = _np(x, np.float32), _np(idx, np.int32), _np(w, np.float32)
        K = idx.size
        if out is None:
            out = np.zeros(self.hidden, np.float32)
        eo = np.empty((K, self.hidden), np.float32) if want_expert_out else None
        self._chk(self.L.fm_moe_decode(self.h, layer, _ptr(x), _ptr(idx), _ptr(w), K, _ptr(out),
                                       _ptr(eo), flags))
        return out, eo

    def moe_decode_dev(self, layer, d_x, d_idx, d_w, K, d_out, d_eo=None, flags=0):
        self._chk(self.L.fm_moe_decode_dev(self.h, layer, d_x, d_idx, d_w, K, d_out, d_eo, flags))

    def moe_decode_step_dev(self, layer0, n_layers, d_x, d_idx, d_w, K, d_out, d_eo=None, flags=0):
        self._chk(self.L.fm_moe_decode_step_dev(self.h, layer0, n_layers, d_x, d_idx, d_w, K,
                                                d_out, d_eo, flags))

    def moe_decode_step_noalloc_dev(self, layer0, n_layers, d_x, d_idx, d_w, K, d_out, flags=0):
        self._chk(self.L.fm_moe_decode_step_noalloc_dev(self.h, layer0, n_layers, d_x, d_idx, d_w, K,
                                                        d_out, flags))

    # ---- prefill
    def moe_prefill(self, layer, X, idx, w, flags=0, out=None):
        X, idx, w = _np(X, np.float32), _np(idx, np.int32), _np(w, np.float32)
        M, K = idx.shape
        if out is None:
            out = np.zeros((M, self.hidden), np.float32)
        self._chk(self.L.fm_moe_prefill(self.h, layer, _ptr(X), _ptr(idx), _ptr(w), M, K,
                                        _ptr(out), flags))
        return out

    def moe_prefill_dev(self, layer, d_X, d_idx, d_w, M, K, d_out, flags=0):
        self._chk(self.L.fm_moe_prefill_dev(self.h, layer, d_X, d_idx, d_w, M, K, d_out, flags))

    def moe_prefill_bf16(self, layer, X_bits, idx, w, flags=0, out=None):
        """X_bits: uint16 [M, hidden], the bfloat16 bit patterns of the activations."""
        X, idx, w = _np(X_bits, np.uint16), _np(idx, np.int32), _np(w, np.float32)
        M, K = idx.shape
        if out is None:
            out = np.zeros((M, self.hidden), np.float32)
        self._chk(self.L.fm_moe_prefill_bf16(self.h, layer, _ptr(X), _ptr(idx), _ptr(w), M, K,
                                             _ptr(out), flags))
        return out

    def moe_prefill_bf16_dev(self, layer, d_X, d_idx, d_w, M, K, d_out, flags=0):
        self._chk(self.L.fm_moe_prefill_bf16_dev(self.h, layer, d_X, d_idx, d_w, M, K, d_out, flags))

    # ---- dense tensors
    def tensor_register(self, W, S, B, out_dim, in_dim, bits=4, group_size=64,
                        scale_dtype=SCALE_BF16):
        W = np.ascontiguousarray(W)
        # S = B = None: an unquantized BF16 tensor [out_dim][in_dim] (bits is ignored)
        S = None if S is None else _np(S, np.uint16)
        B = None if B is None else _np(B, np.uint16)
        t = C.c_int(-1)
        self._chk(self.L.fm_tensor_register(self.h, _ptr(W), _ptr(S), _ptr(B), out_dim, in_dim,
                                            group_size, bits, scale_dtype, C.byref(t)))
        return t.value

    def tensor_adopt(self, d_W, d_S, d_B, out_dim, in_dim, bits=4, group_size=64,
                     scale_dtype=SCALE_BF16):
        t = C.c_int(-1)
        self._chk(self.L.fm_tensor_adopt(self.h, d_W, d_S, d_B, out_dim, in_dim, group_size, bits,
                                         scale_dtype, C.byref(t)))
        return t.value

    def tensor_release(self, t):
        self._chk(self.L.fm_tensor_release(self.h, t))

    def matvec_batch(self, tensors, x, out_dims):
        x = _np(x, np.float32)
        n = len(tensors)
        outs = [np.empty(d, np.float32) for d in out_dims]
        ts = (C.c_int * n)(*tensors)
        ps = (C.c_void_p * n)(*[o.ctypes.data for o in outs])
        self._chk(self.L.fm_matvec_batch(self.h, ts, n, _ptr(x), ps))
        return outs

    def matvec_batch_dev(self, tensors, d_x, d_outs):
        n = len(tensors)
        ts = (C.c_int * n)(*tensors)
        ps = (C.c_void_p * n)(*d_outs)
        self._chk(self.L.fm_matvec_batch_dev(self.h, ts, n, d_x, ps))

    def matvec_batch_route_dev(self, tensors, d_x, d_outs, K, d_seg_score, d_idx, d_w, d_params=None):
        """matvec_batch_dev + route_topk_dev over tensors[0]'s outputs, one launch when it fits."""
        n = len(tensors)
        ts = (C.c_int * n)(*tensors)
        ps = (C.c_void_p * n)(*d_outs)
        self._chk(self.L.fm_matvec_batch_route_dev(self.h, ts, n, d_x, ps, K, d_seg_score, d_idx, d_w,
                                                   d_params))

    def matvec_prefill(self, t, X, out_dim):
        X = _np(X, np.float32)
        M = X.shape[0]
        out = np.empty((M, out_dim), np.float32)
        self._chk(self.L.fm_matvec_prefill(self.h, t, _ptr(X), _ptr(out), M))
        return out

    def matvec_prefill_dev(self, t, d_X, d_out, M):
        self._chk(self.L.fm_matvec_prefill_dev(self.h, t, d_X, d_out, M))

    def matvec_prefill_batch_dev(self, tensors, d_X, d_outs, M):
        n = len(tensors)
        ts = (C.c_int * n)(*tensors)
        outs = (C.c_void_p * n)(*d_outs)
        self._chk(self.L.fm_matvec_prefill_batch_dev(self.h, ts, n, d_X, outs, M))

    # ---- GGUF
    def route_topk_dev(self, d_logits, n_experts, K, d_seg_score, d_idx, d_w, d_params=None):
        self._chk(self.L.fm_route_topk_dev(self.h, d_logits, n_experts, K, d_seg_score, d_idx, d_w,
                                           d_params))

    def layer_tail_dev(self, shared_down, d_h_mid, d_eo, d_params, K, d_shared_gate, d_shared_up,
                       d_next_norm_w, eps, d_hidden_out, d_next_input):
        self._chk(self.L.fm_layer_tail_dev(self.h, shared_down, d_h_mid, d_eo, d_params, K,
                                           d_shared_gate, d_shared_up, d_next_norm_w, eps,
                                           d_hidden_out, d_next_input))

    def moe_decode_tail_dev(self, layer, d_x, d_idx, d_w, K, shared_down, d_h_mid, d_params, d_shared_gate,
                            d_shared_up, d_next_norm_w, eps, d_hidden_out, d_next_input):
        """one layer's routed experts and its tail in one launch (all device pointers)"""
        self._chk(self.L.fm_moe_decode_tail_dev(self.h, layer, d_x, d_idx, d_w, K, shared_down, d_h_mid, d_params,
                                                d_shared_gate, d_shared_up, d_next_norm_w, eps, d_hidden_out,
                                                d_next_input))

    def moe_layer_dev(self, layer, route_tensors, d_x, K, shared_down, d_h_mid, d_next_norm_w, eps, d_logits,
                      d_seg, d_shared_gate, d_shared_up, d_idx, d_w, d_params, d_hidden_out, d_next_input):
        """the MoE half of a layer: routing batch, then routing + experts + tail in one launch"""
        ts = (C.c_int * 4)(*route_tensors)
        self._chk(self.L.fm_moe_layer_dev(self.h, layer, ts, d_x, K, shared_down, d_h_mid, d_next_norm_w, eps,
                                          d_logits, d_seg, d_shared_gate, d_shared_up, d_idx, d_w, d_params,
                                          d_hidden_out, d_next_input))

    def gguf_config(self, n_layers, n_experts, hidden=2048, inter=512,
                    types=(Q4_K, Q4_K, Q6_K)):
        self._chk(self.L.fm_gguf_config(self.h, n_layers, n_experts, hidden, inter, *types))
        self.g_hidden, self.g_inter = hidden, inter

    def gguf_upload_layer(self, layer, gate, up, down):
        gate, up, down = (_np(a, np.uint8).reshape(-1) for a in (gate, up, down))
        self._chk(self.L.fm_gguf_upload_layer(self.h, layer, _ptr(gate), gate.size, _ptr(up), up.size,
                                              _ptr(down), down.size))

    def gguf_adopt_layer(self, layer, d_gate, gate_bytes, d_up, up_bytes, d_down, down_bytes):
        self._chk(self.L.fm_gguf_adopt_layer(self.h, layer, d_gate, gate_bytes, d_up, up_bytes,
                                             d_down, down_bytes))

    def gguf_moe_decode(self, layer, x, idx, w, flags=0, out=None, want_expert_out=True):
        x, idx, w = _np(x, np.float32), _np(idx, np.int32), _np(w, np.float32)
        K = idx.size
        if out is None:
            out = np.zeros(self.g_hidden, np.float32)
        eo = np.empty((K, self.g_hidden), np.float32) if want_expert_out else None
        self._chk(self.L.fm_gguf_moe_decode(self.h, layer, _ptr(x), _ptr(idx), _ptr(w), K,
                                            _ptr(out), _ptr(eo), flags))
        return out, eo

    def gguf_moe_decode_dev(self, layer, d_x, d_idx, d_w, K, d_out, d_eo=None, flags=0):
        self._chk(self.L.fm_gguf_moe_decode_dev(self.h, layer, d_x, d_idx, d_w, K, d_out, d_eo,
                                                flags))

    def gguf_moe_decode_step_dev(self, layer0, n_layers, d_x, d_idx, d_w, K, d_out, d_eo=None,
                                 flags=0):
        self._chk(self.L.fm_gguf_moe_decode_step_dev(self.h, layer0, n_layers, d_x, d_idx, d_w, K,
                                                     d_out, d_eo, flags))

    def gguf_moe_prefill(self, layer, X, idx, w, flags=0, out=None):
        X, idx, w = _np(X, np.float32), _np(idx, np.int32), _np(w, np.float32)
        M, K = idx.shape
        if out is None:
            out = np.zeros((M, self.g_hidden), np.float32)
        self._chk(self.L.fm_gguf_moe_prefill(self.h, layer, _ptr(X), _ptr(idx), _ptr(w), M, K,
                                             _ptr(out), flags))
        return out

    def gguf_moe_prefill_dev(self, layer, d_X, d_idx, d_w, M, K, d_out, flags=0):
        self._chk(self.L.fm_gguf_moe_prefill_dev(self.h, layer, d_X, d_idx, d_w, M, K, d_out,
                                                 flags))

    def gguf_matvec(self, W, ggml_type, x, out_dim, in_dim):
        W, x = _np(W, np.uint8).reshape(-1), _np(x, np.float32)
        out = np.empty(out_dim, np.float32)
        self._chk(self.L.fm_gguf_matvec(self.h, _ptr(W), ggml_type, _ptr(x), _ptr(out), out_dim,
                                        in_dim))
        return out

    # ---- dequant
    def dequant_expert(self, layer, expert, which):
        rows, cols = (self.hidden, self.inter) if which == DOWN else (self.inter, self.hidden)
        codes = np.empty((rows, cols), np.uint8)
        w32 = np.empty((rows, cols), np.float32)
        w16 = np.empty((rows, cols), np.uint16)
        self._chk(self.L.fm_dequant_expert(self.h, layer, expert, which, _ptr(codes), _ptr(w32),
                                           _ptr(w16)))
        return codes, w32, w16

    def dequant_tensor(self, t, out_dim, in_dim):
        codes = np.empty((out_dim, in_dim), np.uint8)
        w32 = np.empty((out_dim, in_dim), np.float32)
        w16 = np.empty((out_dim, in_dim), np.uint16)
        self._chk(self.L.fm_dequant_tensor(self.h, t, _ptr(codes), _ptr(w32), _ptr(w16)))
        return codes, w32, w16

    def embed_lookup_dev(self, t, d_token_ids, n_tokens, d_out):
        self._chk(self.L.fm_embed_lookup_dev(self.h, t, d_token_ids, n_tokens, d_out))

    def embed_lookup(self, t, token_id, in_dim):
        out = np.empty(in_dim, np.float32)
        self._chk(self.L.fm_embed_lookup(self.h, t, int(token_id), _ptr(out)))
        return out

    def gguf_dequant_expert(self, layer, expert, which):
        rows, cols = (self.g_hidden, self.g_inter) if which == DOWN else (self.g_inter, self.g_hidden)
        w32 = np.empty((rows, cols), np.float32)
        self._chk(self.L.fm_gguf_dequant_expert(self.h, layer, expert, which, _ptr(w32)))
        return w32
