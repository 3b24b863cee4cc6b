"""numpy helpers for the reference's packed weight formats: layout arithmetic,
packers and the synthetic-weight recipe of the benchmark configs.

Layouts follow finchmoe/repack_experts.py:76-163 (expert blobs),
finchmoe/quantize_model.py:35-43 (u32 fields), finchmoe/infer.m:1606-1655
(Q4_K / Q6_K blocks).
"""
import numpy as np

GROUP = 64


def expert_layout(hidden=2048, inter=512, bits=3, group=GROUP):
    """Byte offsets of the nine components of one expert and its total size."""
    gu_w = inter * hidden * bits // 8
    gu_s = inter * (hidden // group) * 2
    d_w = hidden * inter * bits // 8
    d_s = hidden * (inter // group) * 2
    names = ["gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b", "down_w", "down_s", "down_b"]
    sizes = [gu_w, gu_s, gu_s, gu_w, gu_s, gu_s, d_w, d_s, d_s]
    lo, o = {}, 0
    for n, s in zip(names, sizes):
        lo[n] = o
        o += s
    lo["expert_size"] = o
    lo["sizes"] = dict(zip(names, sizes))
    return lo


def bf16_trunc(a):
    """fp32 -> bf16 bits by truncation (finchmoe/repack_experts.py:232-234)."""
    return (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)


def bf16_to_f32(u16):
    return (np.asarray(u16, np.uint16).astype(np.uint32) << 16).view(np.float32)


def pack_3bit(codes):
    """8 codes -> 3 bytes, code j at bits 3j..3j+2 (finchmoe/repack_experts.py:242-257)."""
    q = np.ascontiguousarray(codes, np.uint8).reshape(-1, 8).astype(np.uint32)
    acc = np.zeros(q.shape[0], np.uint32)
    for j in range(8):
        acc |= q[:, j] << (3 * j)
    out = np.empty((q.shape[0], 3), np.uint8)
    out[:, 0] = acc & 0xFF
    out[:, 1] = (acc >> 8) & 0xFF
    out[:, 2] = (acc >> 16) & 0xFF
    return out.reshape(-1)


def pack_u32(codes, bits):
    """LSB-first fields of little-endian u32 words (finchmoe/quantize_model.py:35-43)."""
    vpu = 32 // bits
    q = np.ascontiguousarray(codes, np.uint8).reshape(-1, vpu).astype(np.uint32)
    acc = np.zeros(q.shape[0], np.uint32)
    for v in range(vpu):
        acc |= q[:, v] << (v * bits)
    return acc


def pack_codes(codes, bits):
    """Row-major [rows, cols] codes -> packed bytes of the reference layout."""
    if bits == 3:
        return pack_3bit(codes)
    return pack_u32(codes, bits).view(np.uint8)


def synth_scales(rng, shape, dtype="bf16"):
    """scale ~ |N(0, 0.02)| / 3.5 and bias = -3.5 * scale, stored as 16-bit.
    Returns (scale_bits, bias_bits) uint16."""
    s = (np.abs(rng.standard_normal(shape, dtype=np.float32)) * np.float32(0.02)
         / np.float32(3.5)).astype(np.float32)
    b = (np.float32(-3.5) * s).astype(np.float32)
    if dtype == "bf16":
        return bf16_trunc(s), bf16_trunc(b)
    return s.astype(np.float16).view(np.uint16), b.astype(np.float16).view(np.uint16)


def synth_affine_tensor(rng, out_dim, in_dim, bits, dtype="bf16", group=GROUP):
    """Random codes uniform in 0..2^bits-1 + synthetic scales.
    Returns (codes u8 [out,in], W packed bytes, S u16 [out,in/g], B u16)."""
    codes = rng.integers(0, 1 << bits, size=(out_dim, in_dim), dtype=np.uint8)
    S, B = synth_scales(rng, (out_dim, in_dim // group), dtype)
    return codes, pack_codes(codes, bits), S, B


def synth_expert_layer(rng, n_experts, hidden=2048, inter=512, bits=3, dtype="bf16"):
    """One layer_XX.bin worth of synthetic experts: uint8 [n_experts*expert_size]."""
    lo = expert_layout(hidden, inter, bits)
    blob = np.zeros(n_experts * lo["expert_size"], np.uint8)
    for e in range(n_experts):
        base = e * lo["expert_size"]
        for name, rows, cols in (("gate", inter, hidden), ("up", inter, hidden),
                                 ("down", hidden, inter)):
            _, W, S, B = synth_affine_tensor(rng, rows, cols, bits, dtype)
            for part, arr in (("w", W), ("s", S.view(np.uint8).reshape(-1)),
                              ("b", B.view(np.uint8).reshape(-1))):
                o = base + lo[name + "_" + part]
                blob[o:o + arr.size] = arr
    return blob


def expert_views(blob, e, hidden=2048, inter=512, bits=3):
    """Component arrays (W bytes, S u16, B u16) x (gate, up, down) of expert e."""
    lo = expert_layout(hidden, inter, bits)
    base = e * lo["expert_size"]
    out = {}
    for name, rows, cols in (("gate", inter, hidden), ("up", inter, hidden),
                             ("down", hidden, inter)):
        sz = lo["sizes"]
        W = blob[base + lo[name + "_w"]: base + lo[name + "_w"] + sz[name + "_w"]]
        S = blob[base + lo[name + "_s"]: base + lo[name + "_s"] + sz[name + "_s"]].view(np.uint16)
        B = blob[base + lo[name + "_b"]: base + lo[name + "_b"] + sz[name + "_b"]].view(np.uint16)
        out[name] = (W, S.reshape(rows, cols // GROUP), B.reshape(rows, cols // GROUP), rows, cols)
    return out


# ---------------------------------------------------------------- GGUF blocks
def gguf_row_bytes(in_dim, ggml_type):
    return (in_dim // 256) * (144 if ggml_type == 12 else 210)


def synth_gguf_tensor(rng, out_dim, in_dim, ggml_type):
    """Random Q4_K (type 12) or Q6_K (type 14) rows: random codes, random 6-bit
    sub-scales / int8 scales, d and dmin = fp16(|N(0, 0.002)|)."""
    nb = out_dim * (in_dim // 256)
    if ggml_type == 12:
        blk = np.empty((nb, 144), np.uint8)
        d = np.abs(rng.standard_normal((nb, 2), dtype=np.float32) * np.float32(0.002))
        blk[:, 0:4] = d.astype(np.float16).view(np.uint8).reshape(nb, 4)
        blk[:, 4:144] = rng.integers(0, 256, size=(nb, 140), dtype=np.uint8)
    else:
        blk = np.empty((nb, 210), np.uint8)
        blk[:, 0:208] = rng.integers(0, 256, size=(nb, 208), dtype=np.uint8)
        d = np.abs(rng.standard_normal((nb, 1), dtype=np.float32) * np.float32(0.002))
        blk[:, 208:210] = d.astype(np.float16).view(np.uint8).reshape(nb, 2)
    return blk.reshape(-1)


def synth_gguf_layer(rng, n_experts, hidden=2048, inter=512, types=(12, 12, 14)):
    gate = synth_gguf_tensor(rng, n_experts * inter, hidden, types[0])
    up = synth_gguf_tensor(rng, n_experts * inter, hidden, types[1])
    down = synth_gguf_tensor(rng, n_experts * hidden, inter, types[2])
    return gate, up, down


# ---------------------------------------------------------------- routing inputs
def zipf_topk(rng, n_experts, K, s=1.1):
    """K distinct experts, p_e proportional to rank_e^-s under a random rank
    permutation (one draw = one layer of one token)."""
    ranks = rng.permutation(n_experts) + 1
    p = ranks.astype(np.float64) ** (-s)
    p /= p.sum()
    return rng.choice(n_experts, size=K, replace=False, p=p).astype(np.int32)
