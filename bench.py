#!/usr/bin/env python3
"""bench.py — one-GPU benchmark of the quantized-expert hot path.

Default workload (the configuration the headline metric is quoted on): the full 40-layer
routed-expert decode step, batch 1 — all 40 x 256 3-bit g64 experts (14.09 GB) resident in
HBM, per-layer top-8 indices from a Zipf(1.1) distribution with a per-layer rank permutation,
router weights = renormalised softmax of N(0,1) logits at those indices.  A "step" is one
token: one pass of the hot path over all 40 layers.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode_step|decode_layer|gdn|gguf|gguf_chunk|prefill|lm_head|layer_tail|moe_layer|gdn_prefill]

Prints ONE JSON line.  `value` is algorithmic weight bytes per step / wall time per step with
all inputs resident in HBM.  `roofline` prices the dominant kernel against the 8 TB/s HBM
peak using HIP-event durations taken on the library's stream.  `cpu_baseline` times the CPU
oracle (a C restatement of the reference's single-threaded cpu_dequant_matvec expert loop) on
a bounded sample of the same inputs on this box's host.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E peak
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 peak
# HBM bytes per launch of the fused decode kernel on the default workload, from rocprofv3
# --pmc FETCH_SIZE (x2: calibrated against a 1 GiB copy) + WRITE_SIZE.  An OFFLINE constant
# (hardware counters cannot be read from inside this process): the JSON line names the file
# it comes from in roofline.traffic_source, and it is null for any other size.
FUSED_TRAFFIC_BYTES_40L = int((218752.1 * 2 + 2237.6) * 1024)
FUSED_TRAFFIC_SOURCE = "offline constant from profiles/decode_step_3bit_hbm_traffic.md (rocprofv3 --pmc), not measured in this run"
# the same for the one-launch GGUF step (fm_gguf_fused_rows at 40 x 256, top-8)
GGUF_FUSED_TRAFFIC_BYTES_40L = int((322575.7 * 2 + 2148.6) * 1024)
GGUF_FUSED_TRAFFIC_SOURCE = "offline constant from profiles/gguf_step_and_gdn_kernel_trace.md (rocprofv3 --pmc), not measured in this run"
# and for the first of the step's three streaming launches (fm_gguf_stream<Q4_K, 16, gate/up> at 40 x 256, top-8)
GGUF_GATE_UP_TRAFFIC_BYTES_40L = int((185566.3 * 2 + 645.4) * 1024)

H, I, E, K, L = 2048, 512, 256, 8, 40


def _bf16_trunc_bits(t):
    import torch
    return (t.contiguous().view(torch.int32) >> 16).to(torch.int16)


def fill_affine_layer(view, lo, bits, gen, fp16=False):
    """view: uint8 [E, expert_size] on the GPU.  Random codes (all bit patterns are uniform
    codes), scale = bf16(|N(0,0.02)|/3.5), bias = bf16(-3.5*scale) — or both as IEEE halves
    (fp16: the benchmark text's wording; the reference's files hold bf16)."""
    import torch
    view.random_(0, 256, generator=gen)
    for name, rows, cols in (("gate", I, H), ("up", I, H), ("down", H, I)):
        n = rows * (cols // 64)
        s = torch.randn(view.shape[0], n, device=view.device, generator=gen).abs_() * (0.02 / 3.5)
        b = s * -3.5
        for part, val in (("s", s), ("b", b)):
            o = lo[name + "_" + part]
            bits16 = val.to(torch.float16).view(torch.int16) if fp16 else _bf16_trunc_bits(val)
            view[:, o:o + 2 * n] = bits16.contiguous().view(torch.uint8).view(view.shape[0], 2 * n)


def zipf_routing(rng, tokens, layers, n_experts, k):
    """idx [tokens, layers, k] distinct per (token, layer), p_e ~ rank_e^-1.1 with a fixed rank
    permutation per layer; w = renormalised softmax of N(0,1) logits at those indices."""
    idx = np.empty((tokens, layers, k), np.int32)
    for l in range(layers):
        lrng = np.random.default_rng(1000 + l)          # fresh seed per layer
        ranks = lrng.permutation(n_experts) + 1
        p = ranks.astype(np.float64) ** -1.1
        p /= p.sum()
        for t in range(tokens):
            idx[t, l] = lrng.choice(n_experts, size=k, replace=False, p=p)
    logits = rng.standard_normal((tokens, layers, k)).astype(np.float32)
    e = np.exp(logits - logits.max(-1, keepdims=True))
    w = (e / e.sum(-1, keepdims=True)).astype(np.float32)
    return idx, w


def cpu_baseline_decode(blob_t, lo, idx, w, x, budget_s=12.0, bits=3, scale_dtype=0):
    """Oracle expert loop, 1 thread (the reference's path is single-threaded), on (token, layer)
    samples until ~budget_s of CPU time; then a shorter leg with the rows split over 16 threads
    (per-row arithmetic unchanged).  Only the 8 routed experts of each sample are copied back
    from HBM."""
    from oracle import oracle
    oracle.lib()
    es = lo["expert_size"]
    T, Ls = idx.shape[0], idx.shape[1]
    samples = [(t, l) for t in range(T) for l in range(Ls)]

    def leg(nthreads, budget, first):
        done, t_cpu = 0, 0.0
        for (t, l) in samples[first:]:
            sel = idx[t, l]
            mini = np.concatenate([blob_t[l, int(e)].cpu().numpy() for e in sel])
            t0 = time.perf_counter()
            oracle.moe_experts_forward(mini, x[l % x.shape[0]], np.arange(len(sel), dtype=np.int32),
                                       w[t, l], H, I, bits, scale_dtype=scale_dtype, nthreads=nthreads)
            t_cpu += time.perf_counter() - t0
            done += 1
            if t_cpu >= budget:
                break
        return done, t_cpu

    def ref_leg(budget, first):
        """The same blocks through the reference's own compiled CPU functions
        (oracle/_ref/libfm_ref.so: cpu_dequant_matvec x3, cpu_swiglu, cpu_vec_madd, called in the
        order of the CPU expert loop, finchmoe/infer.m:10166-10195).  BF16 scales only (what the
        reference's files hold).  None when the library did not travel with the tree."""
        R = oracle.ref_lib()
        if R is None or scale_dtype != 0:
            return None
        ofs = lo
        g_out, u_out, act = (np.empty(I, np.float32) for _ in range(3))
        e_out, moe = np.empty(H, np.float32), np.zeros(H, np.float32)
        done, t_cpu = 0, 0.0
        for (t, l) in samples[first:]:
            experts = [np.ascontiguousarray(blob_t[l, int(e)].cpu().numpy()) for e in idx[t, l]]
            xv = np.ascontiguousarray(x[l % x.shape[0]], np.float32)
            wv = w[t, l]
            moe[:] = 0.0
            t0 = time.perf_counter()
            for k, eb in enumerate(experts):
                b = eb.ctypes.data
                R.ref_cpu_dequant_matvec(b + ofs["gate_w"], b + ofs["gate_s"], b + ofs["gate_b"], xv.ctypes.data,
                                         g_out.ctypes.data, I, H, 64, bits)
                R.ref_cpu_dequant_matvec(b + ofs["up_w"], b + ofs["up_s"], b + ofs["up_b"], xv.ctypes.data,
                                         u_out.ctypes.data, I, H, 64, bits)
                R.ref_cpu_swiglu(g_out.ctypes.data, u_out.ctypes.data, act.ctypes.data, I)
                R.ref_cpu_dequant_matvec(b + ofs["down_w"], b + ofs["down_s"], b + ofs["down_b"], act.ctypes.data,
                                         e_out.ctypes.data, H, I, 64, bits)
                R.ref_cpu_vec_madd(moe.ctypes.data, e_out.ctypes.data, float(wv[k]), H)
            t_cpu += time.perf_counter() - t0
            done += 1
            if t_cpu >= budget:
                break
        return done, t_cpu, moe.copy(), (t, l)

    bytes_per_layer = len(idx[0, 0]) * es

    def reference_result(port, ref):
        if ref is None or ref[0] == 0:
            return port
        done_r, t_r, moe_ref, (t_last, l_last) = ref
        # the last block once more through the port, outside the timing: the two legs must agree
        mini = np.concatenate([blob_t[l_last, int(e)].cpu().numpy() for e in idx[t_last, l_last]])
        moe_port, _ = oracle.moe_experts_forward(mini, x[l_last % x.shape[0]], np.arange(len(idx[t_last, l_last]), dtype=np.int32),
                                                 w[t_last, l_last], H, I, bits, scale_dtype=scale_dtype)
        same = bool(np.array_equal(moe_ref.view(np.uint32), moe_port.view(np.uint32)))
        out = {
            "value": round(done_r * bytes_per_layer / t_r / 1e9, 4),
            "unit": "GB/s",
            "cores": 1,
            "kind": "reference",
            "us_per_layer": round(t_r / done_r * 1e6, 1),
            "sample": "%d (token, layer) expert blocks of the same workload (8 experts each, %.1f s of CPU "
                      "time) through the reference's own cpu_dequant_matvec / cpu_swiglu / cpu_vec_madd "
                      "(finchmoe/infer.m:1676-1881 compiled gcc -O2 into oracle/_ref/libfm_ref.so), called in "
                      "the order of its CPU expert loop; host has %d logical CPUs" % (done_r, t_r, os.cpu_count()),
            "equals_port_bit_for_bit": same,
            "port": {k: port[k] for k in ("value", "unit", "cores", "us_per_layer", "sample")},
            "rows_over_threads": port["rows_over_threads"],
        }
        return out

    done, t_cpu = leg(1, budget_s, 0)
    many = min(16, os.cpu_count() or 1)
    done_m, t_m = leg(many, min(3.0, budget_s / 4), done)
    port = {
        "value": round(done * bytes_per_layer / t_cpu / 1e9, 4),
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "us_per_layer": round(t_cpu / done * 1e6, 1),
        "sample": "%d (token, layer) expert blocks of the same workload (8 experts each, "
                  "%.1f s of CPU time), oracle/fm_oracle.c gcc -O2, host has %d logical CPUs"
                  % (done, t_cpu, os.cpu_count()),
        "rows_over_threads": {"value": round(done_m * bytes_per_layer / t_m / 1e9, 4), "unit": "GB/s",
                              "cores": many, "us_per_layer": round(t_m / done_m * 1e6, 1),
                              "sample": "%d further blocks, %.1f s" % (done_m, t_m)},
    }
    try:
        return reference_result(port, ref_leg(budget_s, done + done_m))
    except Exception as exc:          # the reference leg must never cost the run its result
        print("bench.py: reference CPU leg skipped: %r" % (exc,), file=sys.stderr)
        return port


def _cpu_leg(run_block, budget_s, max_blocks=None):
    """Calls run_block(i) (which returns the CPU seconds it spent computing, excluding the copy
    of its operands out of HBM) for i = 0, 1, ... until budget_s of CPU time has been used."""
    done, t_cpu = 0, 0.0
    while t_cpu < budget_s and (max_blocks is None or done < max_blocks):
        t_cpu += run_block(done)
        done += 1
    return done, t_cpu


def cpu_baseline_dense(tensors, xs, budget_s=12.0, what="weight set"):
    """The reference's cpu_dequant_matvec (finchmoe/infer.m:1676-1763, compiled into
    oracle/_ref/libfm_ref.so) on the dense tensors of the workload, 1 thread, repeated until
    ~budget_s of CPU time; kind "port" through the oracle's restatement when the reference build
    did not travel with the tree.  tensors: list of sets, a set = list of
    (W, S, B, out_dim, in_dim, bits, x_index) with torch tensors on the GPU."""
    from oracle import oracle
    oracle.lib()
    R = oracle.ref_lib()
    host = {}

    def fetch(i):
        if i not in host:       # one copy per set, outside the timing
            host[i] = [(np.ascontiguousarray(W.cpu().numpy()), np.ascontiguousarray(S.cpu().numpy()).view(np.uint16),
                        np.ascontiguousarray(B.cpu().numpy()).view(np.uint16), od, idim, bits, xi)
                       for (W, S, B, od, idim, bits, xi) in tensors[i]]
        return host[i]

    nbytes = sum(W.numel() + 2 * S.numel() + 2 * B.numel() for (W, S, B, _, _, _, _) in tensors[0])

    def block(i):
        spent = 0.0
        for (W, S, B, od, idim, bits, xi) in fetch(i % len(tensors)):
            x = np.ascontiguousarray(xs[xi], np.float32)
            out = np.empty(od, np.float32)
            t0 = time.perf_counter()
            sp, bp = (None, None) if bits in (10, 11) else (S.ctypes.data, B.ctypes.data)
            if R is not None:
                R.ref_cpu_dequant_matvec(W.ctypes.data, sp, bp, x.ctypes.data, out.ctypes.data, od, idim, 64, bits)
            else:
                oracle.dequant_matvec(W, None if sp is None else S, None if bp is None else B, x, od, idim, bits)
            spent += time.perf_counter() - t0
        return spent

    done, t_cpu = _cpu_leg(block, budget_s)
    return {"value": round(done * nbytes / t_cpu / 1e9, 4), "unit": "GB/s", "cores": 1,
            "kind": "reference" if R is not None else "port", "us_per_step": round(t_cpu / done * 1e6, 1),
            "sample": "%d passes over a %s of the same workload (%.1f s of CPU time) through %s, gcc -O2; host has "
                      "%d logical CPUs" % (done, what, t_cpu,
                                           "the reference's own cpu_dequant_matvec (finchmoe/infer.m:1676-1763, "
                                           "oracle/_ref/libfm_ref.so)" if R is not None else "oracle/fm_oracle.c",
                                           os.cpu_count())}


def cpu_baseline_gguf(layers, idx, w, x, gsl, dsl, budget_s=12.0):
    """Config 4's CPU leg: per (token, layer) block the K routed experts through the reference's
    gguf_cpu_matvec (finchmoe/infer.m:1660-1674, reached as cpu_dequant_matvec with bits 10 = Q4_K
    and 11 = Q6_K), cpu_swiglu and cpu_vec_madd in the order of the CPU expert loop
    (finchmoe/infer.m:10166-10195), 1 thread.  layers: per layer (gate, up, down) uint8 tensors
    [blocks, block_bytes] on the GPU; only the routed experts' rows are copied back."""
    from oracle import oracle
    oracle.lib()
    R = oracle.ref_lib()
    T, Ls = idx.shape[0], idx.shape[1]
    samples = [(t, l) for t in range(T) for l in range(Ls)]
    g_out, u_out, act = (np.empty(I, np.float32) for _ in range(3))
    e_out, moe = np.empty(H, np.float32), np.zeros(H, np.float32)

    def block(i):
        t, l = samples[i % len(samples)]
        g, u, d = layers[l]
        gb, db = I * (H // 256), H * (I // 256)          # blocks per expert
        xv = np.ascontiguousarray(x[(t + l) % x.shape[0]], np.float32)
        experts = [(np.ascontiguousarray(g[int(e) * gb:(int(e) + 1) * gb].cpu().numpy()),
                    np.ascontiguousarray(u[int(e) * gb:(int(e) + 1) * gb].cpu().numpy()),
                    np.ascontiguousarray(d[int(e) * db:(int(e) + 1) * db].cpu().numpy())) for e in idx[t, l]]
        moe[:] = 0.0
        t0 = time.perf_counter()
        if R is not None:
            for k, (ge, ue, de) in enumerate(experts):
                R.ref_cpu_dequant_matvec(ge.ctypes.data, None, None, xv.ctypes.data, g_out.ctypes.data, I, H, 64, 10)
                R.ref_cpu_dequant_matvec(ue.ctypes.data, None, None, xv.ctypes.data, u_out.ctypes.data, I, H, 64, 10)
                R.ref_cpu_swiglu(g_out.ctypes.data, u_out.ctypes.data, act.ctypes.data, I)
                R.ref_cpu_dequant_matvec(de.ctypes.data, None, None, act.ctypes.data, e_out.ctypes.data, H, I, 64, 11)
                R.ref_cpu_vec_madd(moe.ctypes.data, e_out.ctypes.data, float(w[t, l][k]), H)
        else:
            oracle.moe_gguf_forward(np.concatenate([e[0].reshape(-1) for e in experts]),
                                    np.concatenate([e[1].reshape(-1) for e in experts]),
                                    np.concatenate([e[2].reshape(-1) for e in experts]), xv,
                                    np.arange(len(experts), dtype=np.int32), w[t, l], H, I)
        return time.perf_counter() - t0

    done, t_cpu = _cpu_leg(block, budget_s)
    nbytes = idx.shape[2] * (2 * gsl + dsl)
    return {"value": round(done * nbytes / t_cpu / 1e9, 4), "unit": "GB/s", "cores": 1,
            "kind": "reference" if R is not None else "port", "us_per_layer": round(t_cpu / done * 1e6, 1),
            "sample": "%d (token, layer) expert blocks of the same workload (%d GGUF experts each, %.1f s of CPU time) "
                      "through %s, gcc -O2; host has %d logical CPUs"
                      % (done, idx.shape[2], t_cpu,
                         "the reference's own gguf_cpu_matvec / cpu_swiglu / cpu_vec_madd (finchmoe/infer.m:1660-1674, "
                         "1780-1786, oracle/_ref/libfm_ref.so)" if R is not None else "oracle/fm_oracle.c", os.cpu_count())}


def _roofline_hbm(kernel, bytes_per_launch, us_per_launch, launches_per_step=1):
    """roofline object of a bandwidth-bound launch: algorithmic bytes / HIP-event time on the
    library's stream, against the published HBM peak; no counter traffic in this run."""
    ach = bytes_per_launch / (us_per_launch * 1e-6) / 1e9
    return {"bound": "hbm", "kernel": kernel, "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None, "bytes_per_launch": int(bytes_per_launch),
            "us_per_launch": round(us_per_launch, 2), "launches_per_step": launches_per_step}


def run_decode_step(args):
    import torch
    from finchmoe_amd import FinchHip, formats
    dev = torch.device("cuda:0")
    n_layers = args.layers
    bits = args.bits
    lo = formats.expert_layout(H, I, bits)
    es = lo["expert_size"]
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    blob = torch.empty(n_layers, E, es, dtype=torch.uint8, device=dev)
    fp16 = args.scale_dtype == "fp16"
    for l in range(n_layers):
        fill_affine_layer(blob[l], lo, bits, gen, fp16)
    torch.cuda.synchronize()
    ctx = FinchHip(0)
    ctx.experts_config(n_layers, E, H, I, 64, bits, 1 if fp16 else 0)
    for l in range(n_layers):
        ctx.experts_adopt_layer(l, blob[l].data_ptr(), E * es)

    tokens = 256
    rng = np.random.default_rng(7)
    idx, w = zipf_routing(rng, tokens, n_layers, E, K)
    x = rng.standard_normal((n_layers, H)).astype(np.float32)
    d_idx = torch.from_numpy(idx).to(dev)
    d_w = torch.from_numpy(w).to(dev)
    d_x = torch.from_numpy(x).to(dev)
    d_out = torch.empty(n_layers, H, device=dev)
    torch.cuda.synchronize()
    isz = n_layers * K * 4

    def step(t):
        t %= tokens
        ctx.moe_decode_step_dev(0, n_layers, d_x.data_ptr(), d_idx.data_ptr() + t * isz,
                                d_w.data_ptr() + t * isz, K, d_out.data_ptr())

    _ramp_clocks(ctx, step, args.ramp_seconds)
    for t in range(args.warmup):
        step(t)
    ctx.sync()
    torch.cuda.synchronize()
    ctx.timer_start()
    t0 = time.perf_counter()
    for t in range(args.steps):
        step(args.warmup + t)
    ev_ms = ctx.timer_stop()
    ctx.sync()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps

    # The operator is one kernel per step, so the HIP events around the timed region
    # (on the library's stream) give its average launch duration: ev_ms / steps.
    op_us = ev_ms / args.steps * 1e3
    # the phases as separate kernels, each call bracketed by events and waited for
    ctx.kernel_timing(2)
    for t in range(min(args.steps, 300)):
        step(args.warmup + t)
    k1_ms, k2_ms, n = ctx.kernel_timing_read()
    ctx.kernel_timing(0)
    k1_us, k2_us = k1_ms / n * 1e3, k2_ms / n * 1e3

    # per-token latency distribution over 256 consecutive tokens (wall clock incl. sync)
    lat = []
    for t in range(tokens):
        a = time.perf_counter()
        step(t)
        ctx.sync()
        lat.append((time.perf_counter() - a) * 1e6)
    lat = np.array(lat)

    # parity spot check of the last step against nothing cached: finite, non-zero
    out = d_out.cpu().numpy()
    assert np.all(np.isfinite(out)) and np.abs(out).max() > 0

    gu_bytes = 2 * (lo["sizes"]["gate_w"] + 2 * lo["sizes"]["gate_s"])
    bytes_step = n_layers * K * es
    k1_bytes = n_layers * K * gu_bytes
    uniq = len({(l, int(e)) for t in range(tokens) for l in range(n_layers) for e in idx[t, l]})
    res = {
        "metric": "%d-bit expert GEMV HBM GB/s over the %d-layer MoE decode step" % (bits, n_layers),
        "value": round(bytes_step / (ms_per_step * 1e-3) / 1e9, 2),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config 2: %d-layer routed-expert decode step, batch 1, %dx%d %d-bit "
                               "g64 experts resident in HBM (%.2f GB), top-%d Zipf(1.1) routing, "
                               "x~N(0,1) fp32" % (n_layers, n_layers, E, bits, n_layers * E * es / 1e9, K),
                   "hidden": H, "moe_intermediate": I, "experts": E, "top_k": K, "layers": n_layers,
                   "bytes_per_step": bytes_step, "scale_dtype": args.scale_dtype},
        "us_per_step": round(ms_per_step * 1e3, 2),
        "us_per_layer": round(ms_per_step * 1e3 / n_layers, 3),
        "tokens_per_s": round(1e3 / ms_per_step, 1),
        "frac_of_hbm_peak": round(bytes_step / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "event_ms_per_step": round(ev_ms / args.steps, 5),
        "token_latency_us": {"mean": round(float(lat.mean()), 1), "p50": round(float(np.median(lat)), 1),
                             "p99": round(float(np.percentile(lat, 99)), 1)},
        "unique_experts_touched_in_256_tokens": uniq,
        "roofline": {"bound": "hbm", "kernel": "fm_moe_fused_rows<%d,16> (gate/up, down and the sum over the experts in one launch)" % bits,
                     "achieved": round(bytes_step / (op_us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(bytes_step / (op_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": FUSED_TRAFFIC_BYTES_40L if (n_layers, E, K, bits) == (40, 256, 8, 3) else None,
                     "traffic_source": FUSED_TRAFFIC_SOURCE if (n_layers, E, K, bits) == (40, 256, 8, 3) else None,
                     "bytes_per_launch": bytes_step, "us_per_launch": round(op_us, 2)},
        # the same work as three separate kernels (isolated launches, so a little slower
        # than back to back): where the time goes
        "phases_as_kernels_us": {"fm_gate_up_swiglu_lds": round(k1_us, 2),
                                 "fm_down_lds+fm_combine": round(k2_us, 2),
                                 "gate_up_GBps": round(k1_bytes / (k1_us * 1e-6) / 1e9, 1),
                                 "down_GBps": round((bytes_step - k1_bytes) / (k2_us * 1e-6) / 1e9, 1)},
    }
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline_decode(blob, lo, idx, w, x, args.cpu_seconds, bits, 1 if fp16 else 0)
    ctx.close()
    return res


def _finish(res, metric, workload, bytes_step, ms_per_step, args, extra_cfg=None):
    out = {
        "metric": metric, "value": round(bytes_step / (ms_per_step * 1e-3) / 1e9, 2), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic", "config": {"workload": workload, "bytes_per_step": bytes_step},
        "us_per_step": round(ms_per_step * 1e3, 2),
        "frac_of_hbm_peak": round(bytes_step / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
    }
    if extra_cfg:
        out["config"].update(extra_cfg)
    out.update(res)
    return out


def _ramp_clocks(ctx, step, seconds):
    """Untimed: keep the GPU busy with the workload for `seconds` before the W warmup
    steps.  The first launches after an idle period run 10-20 % slower (clock and
    power state ramp), which a warmup counted in steps does not cover when a step
    is ~100 us."""
    t_end = time.perf_counter() + seconds
    t = 0
    while time.perf_counter() < t_end:
        for _ in range(50):
            step(t)
            t += 1
        ctx.sync()
    # the timer calls once, untimed as well: their first call pays one-time costs (symbol lookup in
    # the binding, the runtime's first event read) that would otherwise land inside a short timed run
    ctx.timer_start()
    step(t)
    ctx.timer_stop()
    ctx.sync()


def _timed(ctx, step, args):
    import torch
    _ramp_clocks(ctx, step, args.ramp_seconds)
    for t in range(args.warmup):
        step(t)
    ctx.sync()
    torch.cuda.synchronize()
    ctx.timer_start()
    t0 = time.perf_counter()
    for t in range(args.steps):
        step(args.warmup + t)
    ev_ms = ctx.timer_stop()
    ctx.sync()
    wall = time.perf_counter() - t0
    return wall * 1e3 / args.steps, ev_ms / args.steps


def run_decode_layer(args):
    """config 0: one MoE layer per call, batch 1; calls cycle through 40 distinct layers
    (440 MB > L2, so a call never finds its weights cached by the previous one)."""
    import torch
    from finchmoe_amd import FinchHip, formats
    dev = torch.device("cuda:0")
    lo = formats.expert_layout(H, I, 3)
    es = lo["expert_size"]
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    blob = torch.empty(L, E, es, dtype=torch.uint8, device=dev)
    for l in range(L):
        fill_affine_layer(blob[l], lo, 3, gen)
    ctx = FinchHip(0)
    ctx.experts_config(L, E, H, I, 64, 3, 0)
    for l in range(L):
        ctx.experts_adopt_layer(l, blob[l].data_ptr(), E * es)
    rng = np.random.default_rng(7)
    tokens = 64
    idx, w = zipf_routing(rng, tokens, L, E, K)
    d_idx, d_w = torch.from_numpy(idx).to(dev), torch.from_numpy(w).to(dev)
    d_x = torch.randn(L, H, device=dev)
    d_out = torch.empty(L, H, device=dev)
    torch.cuda.synchronize()

    def step(t):
        l, tok = t % L, (t // L) % tokens
        o = (tok * L + l) * K * 4
        ctx.moe_decode_dev(l, d_x.data_ptr() + l * H * 4, d_idx.data_ptr() + o, d_w.data_ptr() + o, K,
                           d_out.data_ptr() + l * H * 4)

    ms, ev = _timed(ctx, step, args)
    ctx.kernel_timing(2)   # the phases as separate kernels, isolated launches
    for t in range(args.steps):
        step(t)
    k1, k2, n = ctx.kernel_timing_read()
    ctx.kernel_timing(0)
    res = {"phases_as_kernels_us": {"fm_gate_up_swiglu_lds": round(k1 / n * 1e3, 2),
                                    "fm_down_lds+fm_combine": round(k2 / n * 1e3, 2)},
           "event_ms_per_step": round(ev, 5), "us_per_layer": round(ms * 1e3, 3),
           "roofline": _roofline_hbm("fm_moe_fused_rows<3,16> (one layer per launch: latency-bound)", K * es, ev * 1e3)}
    if not args.no_cpu:
        x = d_x.cpu().numpy()
        res["cpu_baseline"] = cpu_baseline_decode(blob, lo, idx, w, x, args.cpu_seconds, 3, 0)
    ctx.close()
    return _finish(res, "3-bit expert GEMV HBM GB/s, one MoE layer per call", "config 0: single MoE layer, decode "
                   "batch 1, hidden 2048, 256 experts, top-8, 3-bit g64; calls cycle over 40 layers",
                   K * es, ms, args)


def run_gdn(args):
    """config 1: dense 4-bit GatedDeltaNet projections, batch 1, 40 independent weight sets."""
    import torch
    from finchmoe_amd import FinchHip
    dev = torch.device("cuda:0")
    ctx = FinchHip(0)
    gen = torch.Generator(device=dev)
    gen.manual_seed(99)
    sets = []
    keep = []

    def tensor(out_dim, in_dim):
        W = torch.empty(out_dim * in_dim // 2, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
        s = torch.randn(out_dim * (in_dim // 64), device=dev, generator=gen).abs_() * (0.02 / 3.5)
        b = s * -3.5
        S, B = _bf16_trunc_bits(s), _bf16_trunc_bits(b)
        keep.extend([W, S, B])
        return ctx.tensor_adopt(W.data_ptr(), S.data_ptr(), B.data_ptr(), out_dim, in_dim, 4)

    nsets = 40
    for _ in range(nsets):
        sets.append((tensor(8192, 2048), tensor(4096, 2048), tensor(2048, 4096)))
    # the same tensors for the CPU leg: keep[] holds (W, S, B) of every tensor in order
    cpu_sets = [[(keep[9 * i + 0], keep[9 * i + 1], keep[9 * i + 2], 8192, 2048, 4, 0),
                 (keep[9 * i + 3], keep[9 * i + 4], keep[9 * i + 5], 4096, 2048, 4, 0),
                 (keep[9 * i + 6], keep[9 * i + 7], keep[9 * i + 8], 2048, 4096, 4, 1)] for i in range(nsets)]
    d_x = torch.randn(2048, device=dev)
    d_y = torch.randn(4096, device=dev)
    oq, oz, oo = (torch.empty(n, device=dev) for n in (8192, 4096, 2048))
    torch.cuda.synchronize()

    def step(t):
        q, z, o = sets[t % nsets]
        ctx.matvec_batch_dev([q, z], d_x.data_ptr(), [oq.data_ptr(), oz.data_ptr()])
        ctx.matvec_batch_dev([o], d_y.data_ptr(), [oo.data_ptr()])

    ms, ev = _timed(ctx, step, args)
    bytes_set = 12288 * 1152 + 2048 * (2048 + 256)
    res = {"event_ms_per_step": round(ev, 5),
           "roofline": _roofline_hbm("fm_dense_stream<4,16,1> (in_proj qkv+z) + fm_dense_gemv<4,32> (out_proj): the two "
                                     "launches of a weight set, latency-bound", bytes_set, ev * 1e3, 2)}
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline_dense(cpu_sets, [d_x.cpu().numpy(), d_y.cpu().numpy()], args.cpu_seconds,
                                                 "weight set (in_proj qkv + z, out_proj)")
    ctx.close()
    return _finish(res, "dense 4-bit GatedDeltaNet projection GEMV HBM GB/s", "config 1: in_proj_qkv+z "
                   "2048->12288 and out_proj 4096->2048, 4-bit g64, batch 1, 40 weight sets cycled",
                   bytes_set, ms, args)


def run_lm_head(args):
    """Next row after the expert path: the [vocab 248320, 2048] output projection, batch 1, three
    weight sets cycled: 8-bit affine (finchmoe/infer.m:5728-5760) or, with --lm-format q4k / q6k,
    the GGUF block formats of a GGUF model's output.weight (finchmoe/infer.m:5738-5746)."""
    import torch
    from finchmoe_amd import FinchHip
    dev = torch.device("cuda:0")
    ctx = FinchHip(0)
    gen = torch.Generator(device=dev)
    gen.manual_seed(11)
    V, D = 248320, 2048
    keep, sets = [], []
    fmt = args.lm_format
    for _ in range(3):
        if fmt == "affine8":
            W = torch.empty(V * D, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
            s = torch.randn(V * (D // 64), device=dev, generator=gen).abs_() * (0.02 / 127.5)
            b = s * -127.5
            S, B = _bf16_trunc_bits(s), _bf16_trunc_bits(b)
            keep.extend([W, S, B])
            sets.append(ctx.tensor_adopt(W.data_ptr(), S.data_ptr(), B.data_ptr(), V, D, 8))
        else:
            bsz, n_d, d_off, bits = (144, 2, 0, 10) if fmt == "q4k" else (210, 1, 208, 11)
            W = torch.empty(V * (D // 256), bsz, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
            d = (torch.randn(V * (D // 256), n_d, device=dev, generator=gen).abs_() * 0.002).to(torch.float16)
            W[:, d_off:d_off + 2 * n_d] = d.view(torch.uint8)
            keep.append(W)
            sets.append(ctx.tensor_adopt(W.data_ptr(), None, None, V, D, bits))
    d_x = torch.randn(D, device=dev)
    d_o = torch.empty(V, device=dev)
    torch.cuda.synchronize()

    def step(t):
        ctx.matvec_batch_dev([sets[t % 3]], d_x.data_ptr(), [d_o.data_ptr()])

    ms, ev = _timed(ctx, step, args)
    assert torch.isfinite(d_o).all()
    if fmt == "affine8":
        bytes_set = V * D + 2 * V * (D // 64) * 2
        kernel = "fm_dense_stream<8,16,1>"
    else:
        bytes_set = V * (D // 256) * (144 if fmt == "q4k" else 210)
        kernel = "fm_gguf_stream<Q4_K,16,down> on one dense tensor" if fmt == "q4k" else "fm_gguf_matvec_rows_k<Q6_K,16>"
    res = {"event_ms_per_step": round(ev, 5), "roofline": _roofline_hbm(kernel, bytes_set, ev * 1e3)}
    if not args.no_cpu:
        # a bounded sample: the first 8192 rows of a set (the per-row arithmetic does not depend on the row)
        rows = 8192
        if fmt == "affine8":
            sub = [[(keep[3 * i][:rows * D], keep[3 * i + 1][:rows * (D // 64)], keep[3 * i + 2][:rows * (D // 64)], rows, D, 8, 0)]
                   for i in range(3)]
        else:
            empty = torch.empty(0, dtype=torch.int16)
            sub = [[(keep[i][:rows * (D // 256)].reshape(-1), empty, empty, rows, D, 10 if fmt == "q4k" else 11, 0)]
                   for i in range(3)]
        res["cpu_baseline"] = cpu_baseline_dense(sub, [d_x.cpu().numpy()], args.cpu_seconds,
                                                 "%d-row slice of the projection" % rows)
    ctx.close()
    return _finish(res, "%s output projection GEMV HBM GB/s" % {"affine8": "8-bit", "q4k": "GGUF Q4_K", "q6k": "GGUF Q6_K"}[fmt],
                   "lm_head 2048->248320, %s, batch 1, 3 weight sets cycled" % {"affine8": "8-bit g64", "q4k": "Q4_K", "q6k": "Q6_K"}[fmt],
                   bytes_set, ms, args)


def run_layer_tail(args):
    """Next row after the expert path: shared-expert down projection + combine with residual +
    next layer's RMS norm in one launch (finchmoe/infer.m:9608-9760), 40 layers' tensors cycled."""
    import torch
    from finchmoe_amd import FinchHip
    dev = torch.device("cuda:0")
    ctx = FinchHip(0)
    gen = torch.Generator(device=dev)
    gen.manual_seed(13)
    SI = 512
    keep, ts = [], []
    for _ in range(40):
        W = torch.empty(H * SI // 2, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
        s = torch.randn(H * (SI // 64), device=dev, generator=gen).abs_() * (0.02 / 7.5)
        S, B = _bf16_trunc_bits(s), _bf16_trunc_bits(s * -7.5)
        keep.extend([W, S, B])
        ts.append(ctx.tensor_adopt(W.data_ptr(), S.data_ptr(), B.data_ptr(), H, SI, 4))
    h_mid, eo = torch.randn(H, device=dev), torch.randn(K, H, device=dev)
    params = torch.zeros(10, device=dev)
    params[:K] = 1.0 / K
    sg, su = torch.randn(SI, device=dev), torch.randn(SI, device=dev)
    nw = torch.ones(H, device=dev).to(torch.bfloat16)
    hid, nxt = torch.empty(H, device=dev), torch.empty(H, device=dev)
    torch.cuda.synchronize()

    def step(t):
        ctx.layer_tail_dev(ts[t % 40], h_mid.data_ptr(), eo.data_ptr(), params.data_ptr(), K,
                           sg.data_ptr(), su.data_ptr(), nw.data_ptr(), 1e-6, hid.data_ptr(),
                           nxt.data_ptr())

    ms, ev = _timed(ctx, step, args)
    assert torch.isfinite(nxt).all()
    bytes_call = H * SI // 2 + 2 * H * (SI // 64) * 2 + (K + 4) * H * 4
    res = {"event_ms_per_step": round(ev, 5),
           "roofline": _roofline_hbm("fm_layer_tail (latency-bound)", bytes_call, ev * 1e3)}
    ctx.close()
    return _finish(res, "layer tail (shared down + combine + residual + RMS norm) GB/s",
                   "one launch per layer: 4-bit [2048,512] shared down projection, K=8 combine, "
                   "next-layer norm; 40 tensors cycled", bytes_call, ms, args)


def run_moe_layer(args):
    """The MoE half of every layer without a host round trip, one token per step: routing and
    shared-expert GEMVs (8-bit gate [256,2048] and shared-gate score, 4-bit shared gate/up
    [512,2048]) -> softmax/top-8 -> routed experts -> shared down + combine + residual + next
    layer's norm (finchmoe/infer.m:9285-9760), layer l+1 reading what layer l wrote.  Three
    launches per layer (the GEMV batch's last workgroup routes); with --graph the whole token is one captured HIP graph."""
    import ctypes as C
    import torch
    from finchmoe_amd import FinchHip, formats
    dev = torch.device("cuda:0")
    n_layers = args.layers
    lo = formats.expert_layout(H, I, 3)
    es = lo["expert_size"]
    gen = torch.Generator(device=dev)
    gen.manual_seed(99)
    blob = torch.empty(n_layers, E, es, dtype=torch.uint8, device=dev)
    for l in range(n_layers):
        fill_affine_layer(blob[l], lo, 3, gen)
    ctx = FinchHip(0)
    ctx.experts_config(n_layers, E, H, I, 64, 3, 0)
    for l in range(n_layers):
        ctx.experts_adopt_layer(l, blob[l].data_ptr(), E * es)
    keep, dense_bytes = [], 0

    def tensor(rows, cols, bits, gain):
        nonlocal dense_bytes
        W = torch.empty(rows * cols * bits // 8, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
        half = ((1 << bits) - 1) / 2.0
        sc = torch.randn(rows * (cols // 64), device=dev, generator=gen).abs_() * (gain / half)
        S, B = _bf16_trunc_bits(sc), _bf16_trunc_bits(sc * -half)
        keep.extend([W, S, B])
        dense_bytes += W.numel() + 4 * S.numel()
        return ctx.tensor_adopt(W.data_ptr(), S.data_ptr(), B.data_ptr(), rows, cols, bits)

    layers = []
    for l in range(n_layers):
        layers.append((tensor(E, H, 8, 0.05), tensor(1, H, 8, 0.02), tensor(I, H, 4, 0.02),
                       tensor(I, H, 4, 0.02), tensor(H, I, 4, 0.02)))
    x0 = torch.randn(H, device=dev)
    hid = [torch.empty(H, device=dev) for _ in range(2)]
    xin = [torch.empty(H, device=dev) for _ in range(2)]
    d_log, d_seg = torch.empty(E, device=dev), torch.empty(1, device=dev)
    d_sg, d_su = torch.empty(I, device=dev), torch.empty(I, device=dev)
    d_idx = torch.empty(K, dtype=torch.int32, device=dev)
    d_w, d_p = torch.empty(K, device=dev), torch.empty(10, device=dev)
    d_moe, d_eo = torch.empty(H, device=dev), torch.empty(K, H, device=dev)
    nw = torch.ones(H, device=dev).to(torch.bfloat16)
    torch.cuda.synchronize()

    # --forms three-launches: experts and tail as two launches (the form a captured graph takes)
    three = "three-launches" in args.forms or bool(args.graph)

    def token():
        for l in range(n_layers):
            t_gate, t_seg, t_sg, t_su, t_sd = layers[l]
            x = x0 if l == 0 else xin[(l - 1) & 1]
            h_mid = x0 if l == 0 else hid[(l - 1) & 1]
            if not three:
                # two launches: the routing batch; routing + experts + tail (bit for bit the three below)
                ctx.moe_layer_dev(l, [t_gate, t_seg, t_sg, t_su], x.data_ptr(), K, t_sd, h_mid.data_ptr(),
                                  nw.data_ptr(), 1e-6, d_log.data_ptr(), d_seg.data_ptr(), d_sg.data_ptr(),
                                  d_su.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), d_p.data_ptr(),
                                  hid[l & 1].data_ptr(), xin[l & 1].data_ptr())
                continue
            ctx.matvec_batch_route_dev([t_gate, t_seg, t_sg, t_su], x.data_ptr(),
                                       [d_log.data_ptr(), d_seg.data_ptr(), d_sg.data_ptr(), d_su.data_ptr()],
                                       K, d_seg.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), d_p.data_ptr())
            if three:
                # no buffer for the per-expert vectors: the experts' sum goes to d_moe, and the tail
                # takes it as it is (K = 0 with a vector)
                ctx.moe_decode_dev(l, x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K, d_moe.data_ptr(), None)
                ctx.layer_tail_dev(t_sd, h_mid.data_ptr(), d_moe.data_ptr(), d_p.data_ptr(), 0, d_sg.data_ptr(),
                                   d_su.data_ptr(), nw.data_ptr(), 1e-6, hid[l & 1].data_ptr(), xin[l & 1].data_ptr())
            else:
                # the experts and the tail in one launch (bit for bit the two calls above)
                ctx.moe_decode_tail_dev(l, x.data_ptr(), d_idx.data_ptr(), d_w.data_ptr(), K, t_sd, h_mid.data_ptr(),
                                        d_p.data_ptr(), d_sg.data_ptr(), d_su.data_ptr(), nw.data_ptr(), 1e-6,
                                        hid[l & 1].data_ptr(), xin[l & 1].data_ptr())

    token()
    ctx.sync()
    ref = xin[(n_layers - 1) & 1].clone()
    assert torch.isfinite(ref).all() and ref.abs().max() > 0
    step = lambda t: token()
    if args.graph:
        hip = C.CDLL("libamdhip64.so")
        stream, graph, gexec = C.c_void_p(ctx.stream()), C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(stream, C.c_int(2)) == 0
        token()
        assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
        step = lambda t: hip.hipGraphLaunch(gexec, stream)
    ms, ev = _timed(ctx, step, args)
    ctx.sync()
    assert torch.equal(xin[(n_layers - 1) & 1], ref)      # same inputs, same result on every step
    nl_launch = 3 if three else 2
    res = {"us_per_layer": round(ms * 1e3 / n_layers, 2), "launches_per_layer": nl_launch,
           "graph": bool(args.graph), "event_ms_per_step": round(ev, 5),
           "roofline": _roofline_hbm(("fm_dense_gemv_mixed + fm_moe_fused_rows<3,16> + fm_layer_tail per layer "
                                      "(three dependent launches, latency-bound)") if three else
                                     ("fm_dense_gemv_mixed + fm_moe_fused_rows_tail<3,16> (routing, experts, tail) per layer "
                                      "(two dependent launches, latency-bound)"), n_layers * K * es + dense_bytes,
                                     ev * 1e3, nl_launch * n_layers)}
    ctx.close()
    return _finish(res, "MoE half of a layer on the device, GB/s over a %d-layer token" % n_layers,
                   "routing + shared-expert GEMVs, top-8, routed 3-bit experts (router-chosen), shared "
                   "down + combine + norm; %d layers chained, %s" % (n_layers, "one HIP graph per token"
                                                                     if args.graph else "eager launches"),
                   n_layers * K * es + dense_bytes, ms, args)


def run_gdn_prefill(args):
    """config 1's tensors against M positions (M = --chunk, the reference's
    gpu_encode_prefill_matvec): in_proj_qkv [8192,2048] and in_proj_z [4096,2048] from X[M,2048],
    out_proj [2048,4096] from Y[M,4096]; 4-bit g64.  From 16 positions on the products run on the
    matrix cores."""
    import torch
    from finchmoe_amd import FinchHip
    dev = torch.device("cuda:0")
    M = args.chunk
    ctx = FinchHip(0)
    gen = torch.Generator(device=dev)
    gen.manual_seed(21)
    keep, sets, nsets = [], [], 8

    def tensor(rows, cols):
        W = torch.empty(rows * cols // 2, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
        sc = torch.randn(rows * (cols // 64), device=dev, generator=gen).abs_() * (0.02 / 7.5)
        S, B = _bf16_trunc_bits(sc), _bf16_trunc_bits(sc * -7.5)
        keep.extend([W, S, B])
        return ctx.tensor_adopt(W.data_ptr(), S.data_ptr(), B.data_ptr(), rows, cols, 4)

    for _ in range(nsets):
        sets.append((tensor(8192, 2048), tensor(4096, 2048), tensor(2048, 4096)))
    X, Y = torch.randn(M, 2048, device=dev), torch.randn(M, 4096, device=dev)
    oq, oz, oo = (torch.empty(M, 8192, device=dev), torch.empty(M, 4096, device=dev),
                  torch.empty(M, 2048, device=dev))
    torch.cuda.synchronize()

    def step(t):
        tq, tz, to = sets[t % nsets]
        ctx.matvec_prefill_batch_dev([tq, tz], X.data_ptr(), [oq.data_ptr(), oz.data_ptr()], M)
        ctx.matvec_prefill_dev(to, Y.data_ptr(), oo.data_ptr(), M)

    ms, ev = _timed(ctx, step, args)
    assert torch.isfinite(oo).all() and torch.isfinite(oq).all()
    flops = 2.0 * M * (12288 * 2048 + 2048 * 4096)
    res = {"tflops": round(flops / (ms * 1e-3) / 1e12, 2),
           "frac_of_bf16_mfma_peak": round(flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
           "event_ms_per_step": round(ev, 5),
           "roofline": {"bound": "mfma", "kernel": "fm_pf_gemm<PF_DENSE,4> (+ fm_pf_dense_prep)",
                        "achieved": round(flops / (ev * 1e-3) / 1e12, 2), "peak": MFMA_BF16_PEAK_TFLOPS,
                        "unit": "TFLOP/s", "frac": round(flops / (ev * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                        "traffic": None, "flops_per_step": flops, "us_per_step": round(ev * 1e3, 2)}}
    ctx.close()
    return _finish(res, "dense 4-bit GatedDeltaNet projections against %d positions" % M,
                   "config 1's weight set (qkv 8192x2048, z 4096x2048, out_proj 2048x4096, 4-bit g64) "
                   "x %d positions, qkv and z in one call, %d sets cycled" % (M, nsets),
                   18874368, ms, args, {"flops_per_step": flops})


def run_gguf(args):
    """config 4: GGUF experts (Q4_K gate/up, Q6_K down), 40-layer decode step, batch 1."""
    import torch
    from finchmoe_amd import FinchHip
    dev = torch.device("cuda:0")
    n_layers = args.layers
    gsl, dsl = I * (H // 256) * 144, H * (I // 256) * 210
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    ctx = FinchHip(0)
    ctx.gguf_config(n_layers, E, H, I)
    keep = []

    def slab(nblocks, bsz, d_off, n_d):
        t = torch.empty(nblocks, bsz, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
        d = (torch.randn(nblocks, n_d, device=dev, generator=gen).abs_() * 0.002).to(torch.float16)
        t[:, d_off:d_off + 2 * n_d] = d.view(torch.uint8)
        return t

    for l in range(n_layers):
        g = slab(E * I * (H // 256), 144, 0, 2)
        u = slab(E * I * (H // 256), 144, 0, 2)
        d = slab(E * H * (I // 256), 210, 208, 1)
        keep.extend([g, u, d])
        ctx.gguf_adopt_layer(l, g.data_ptr(), g.numel(), u.data_ptr(), u.numel(), d.data_ptr(), d.numel())
    rng = np.random.default_rng(7)
    tokens = max(64, args.chunk) if args.workload == "gguf_chunk" else 64
    idx, w = zipf_routing(rng, tokens, n_layers, E, K)
    if args.workload == "gguf_chunk":
        # the chunked-prefill variant of config 4: M positions of one layer per call (grouped
        # products from 32 positions on, per-position products below, as the reference runs
        # them; --forms per-position forces the latter), the layer changes from call to call
        M = args.chunk if args.chunk <= tokens else 8
        per_position = "per-position" in args.forms
        c_idx = torch.from_numpy(np.ascontiguousarray(idx.transpose(1, 0, 2))).to(dev)   # [layer][token][k]
        c_w = torch.from_numpy(np.ascontiguousarray(w.transpose(1, 0, 2))).to(dev)
        c_x = torch.randn(M, H, device=dev)
        c_out = torch.empty(M, H, device=dev)
        torch.cuda.synchronize()
        lsz = tokens * K * 4

        def cstep(t):
            l = t % n_layers
            ctx.gguf_moe_prefill_dev(l, c_x.data_ptr(), c_idx.data_ptr() + l * lsz, c_w.data_ptr() + l * lsz,
                                     M, K, c_out.data_ptr())

        ms, ev = _timed(ctx, cstep, args)
        assert torch.isfinite(c_out).all()
        grouped = M >= 32 and M * K >= 2 * E and not per_position      # the library's own condition
        # grouped products read an expert once per group of its positions: priced on the distinct
        # experts of a chunk; per-position products stream every routed expert once per position
        uniq = float(np.mean([len(set(idx[:M, l].reshape(-1).tolist())) for l in range(n_layers)]))
        rbytes = uniq * (2 * gsl + dsl) if grouped else M * K * (2 * gsl + dsl)
        # (per-position products: the library takes the one launch up to 8 positions and the three
        # streaming launches beyond)
        one = not grouped and not any(f in args.forms for f in ("gguf-phases", "plain-gguf")) and \
            (M <= 8 or "gguf-one-launch" in args.forms)
        cres = {"event_ms_per_step": round(ev, 5),
                "roofline": _roofline_hbm("fm_gq_gate_up + fm_gq_down + fm_pf_combine (grouped products; bytes of the "
                                          "chunk's distinct experts)" if grouped else
                                          "fm_gguf_fused_rows (one launch, one group per position)" if one else
                                          "fm_gguf_stream<Q4_K gate/up> + fm_gguf_stream<Q6_K down> + fm_gguf_combine "
                                          "(one group per position)", rbytes, ev * 1e3, 4 if grouped else 1 if one else 3)}
        if grouped:
            flops = 2.0 * M * K * 3 * H * I
            cres["tflops"] = round(flops / (ev * 1e-3) / 1e12, 2)
            cres["frac_of_bf16_mfma_peak"] = round(flops / (ev * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)
        if not args.no_cpu:
            cres["cpu_baseline"] = cpu_baseline_gguf([keep[3 * l:3 * l + 3] for l in range(n_layers)], idx[:M], w[:M],
                                                     c_x.cpu().numpy(), gsl, dsl, args.cpu_seconds)
        ctx.close()
        return _finish(cres,
                       "GGUF Q4_K/Q6_K expert GEMV HBM GB/s, %d-position chunk of one layer" % M,
                       "config 4, chunk variant: %d positions x top-8 Zipf(1.1) on one of %d GGUF layers "
                       "(Q4_K gate/up, Q6_K down), %s products" % (M, n_layers, "grouped" if grouped else "per-position"),
                       M * K * (2 * gsl + dsl), ms, args)
    d_idx, d_w = torch.from_numpy(idx).to(dev), torch.from_numpy(w).to(dev)
    d_x = torch.randn(n_layers, H, device=dev)
    d_out = torch.empty(n_layers, H, device=dev)
    torch.cuda.synchronize()
    isz = n_layers * K * 4

    def step(t):
        t %= tokens
        ctx.gguf_moe_decode_step_dev(0, n_layers, d_x.data_ptr(), d_idx.data_ptr() + t * isz,
                                     d_w.data_ptr() + t * isz, K, d_out.data_ptr())

    ms, ev = _timed(ctx, step, args)
    ctx.kernel_timing(True)
    for t in range(args.steps):
        step(t)
    k1, k2, n = ctx.kernel_timing_read()
    ctx.kernel_timing(0)
    assert torch.isfinite(d_out).all()
    # (the library's own choice: one launch up to 13 layers, three streaming launches beyond)
    phases = any(f in args.forms for f in ("gguf-phases", "plain-gguf")) or (n_layers > 13 and "gguf-one-launch" not in args.forms)
    res = {"kernels_us": {"fm_gguf_gate_up (as three launches)": round(k1 / n * 1e3, 2),
                          "fm_gguf_down+combine (as three launches)": round(k2 / n * 1e3, 2)},
           "event_ms_per_step": round(ev, 5), "us_per_layer": round(ms * 1e3 / n_layers, 3),
           "tokens_per_s": round(1e3 / ms, 1), "launches_per_step": 3 if phases else 1}
    if phases:
        # the dominant kernel: the Q4_K gate/up stream (its own events, isolated launches)
        res["roofline"] = _roofline_hbm("fm_gguf_stream<Q4_K,16,gate/up> (first of the step's three launches)",
                                        n_layers * K * 2 * gsl, k1 / n * 1e3)
        if (n_layers, E, K) == (40, 256, 8):
            res["roofline"]["traffic"] = GGUF_GATE_UP_TRAFFIC_BYTES_40L
            res["roofline"]["traffic_source"] = GGUF_FUSED_TRAFFIC_SOURCE
    else:
        # the step is one launch: HIP events around the timed region on the library's stream
        res["roofline"] = _roofline_hbm("fm_gguf_fused_rows<Q6_K,16,8> (the step's one launch)",
                                        n_layers * K * (2 * gsl + dsl), ev * 1e3)
        if (n_layers, E, K) == (40, 256, 8):
            res["roofline"]["traffic"] = GGUF_FUSED_TRAFFIC_BYTES_40L
            res["roofline"]["traffic_source"] = GGUF_FUSED_TRAFFIC_SOURCE
    res["roofline"]["step"] = {"bytes": n_layers * K * (2 * gsl + dsl), "us": round(ev * 1e3, 2),
                               "frac": round(n_layers * K * (2 * gsl + dsl) / (ev * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline_gguf([keep[3 * l:3 * l + 3] for l in range(n_layers)], idx, w,
                                                d_x.cpu().numpy(), gsl, dsl, args.cpu_seconds)
    ctx.close()
    return _finish(res, "GGUF Q4_K/Q6_K expert GEMV HBM GB/s over the %d-layer decode step" % n_layers,
                   "config 4: %dx%d GGUF experts (Q4_K gate/up, Q6_K down) resident, top-8 Zipf(1.1), batch 1"
                   % (n_layers, E), n_layers * K * (2 * gsl + dsl), ms, args)


def run_prefill(args):
    """config 3: chunked prefill of M positions on one layer (M = --chunk)."""
    import torch
    from finchmoe_amd import FinchHip, formats
    dev = torch.device("cuda:0")
    M = args.chunk
    bits = args.bits
    lo = formats.expert_layout(H, I, bits)
    es = lo["expert_size"]
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    nl = 8
    blob = torch.empty(nl, E, es, dtype=torch.uint8, device=dev)
    fp16 = args.scale_dtype == "fp16"
    for l in range(nl):
        fill_affine_layer(blob[l], lo, bits, gen, fp16)
    ctx = FinchHip(0)
    ctx.experts_config(nl, E, H, I, 64, bits, 1 if fp16 else 0)
    for l in range(nl):
        ctx.experts_adopt_layer(l, blob[l].data_ptr(), E * es)
    rng = np.random.default_rng(7)
    idx, w = zipf_routing(rng, M, nl, E, K)          # [M, nl, K]
    if args.prefill_experts:
        # profile buckets: uniform routing over the first N experts (N = 16: 256 positions per
        # expert of a 512-position chunk, every item full; N = 256 with --chunk 128: 4 per expert)
        n_e = max(K, min(E, args.prefill_experts))
        for t in range(M):
            for l in range(nl):
                idx[t, l] = rng.permutation(n_e)[:K]
    idx = np.ascontiguousarray(idx.transpose(1, 0, 2))
    w = np.ascontiguousarray(w.transpose(1, 0, 2))
    d_idx, d_w = torch.from_numpy(idx).to(dev), torch.from_numpy(w).to(dev)
    d_Xb = torch.randn(M, H, device=dev).to(torch.bfloat16)     # x ~ N(0,1) bf16
    d_X = d_Xb.to(torch.float32)                                # the same values as fp32
    d_out = torch.empty(M, H, device=dev)
    torch.cuda.synchronize()
    as_bf16 = args.x_dtype == "bf16"

    def step(t):
        l = t % nl
        if as_bf16:
            ctx.moe_prefill_bf16_dev(l, d_Xb.data_ptr(), d_idx.data_ptr() + l * M * K * 4,
                                     d_w.data_ptr() + l * M * K * 4, M, K, d_out.data_ptr())
        else:
            ctx.moe_prefill_dev(l, d_X.data_ptr(), d_idx.data_ptr() + l * M * K * 4,
                                d_w.data_ptr() + l * M * K * 4, M, K, d_out.data_ptr())

    ms, ev = _timed(ctx, step, args)
    flops = M * K * 3 * 2 * H * I
    uniq = float(np.mean([len(set(idx[l].reshape(-1).tolist())) for l in range(nl)]))
    res = {"tflops": round(flops / (ms * 1e-3) / 1e12, 2),
           "frac_of_bf16_mfma_peak": round(flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
           "unique_experts_per_chunk": uniq, "event_ms_per_step": round(ev, 5),
           "positions_per_s": round(M / (ms * 1e-3), 1)}
    if not args.no_cpu:
        # the reference runs a chunk position by position: (position, layer) expert blocks
        cpu_idx = np.ascontiguousarray(idx.transpose(1, 0, 2))        # [position][layer][k]
        cpu_w = np.ascontiguousarray(w.transpose(1, 0, 2))
        res["cpu_baseline"] = cpu_baseline_decode(blob, lo, cpu_idx, cpu_w, d_X.cpu().numpy(), args.cpu_seconds, bits,
                                                  1 if fp16 else 0)
        res["cpu_baseline"]["positions_per_s"] = round(1e6 / res["cpu_baseline"]["us_per_layer"], 2)
    ctx.close()
    out = _finish(res, "chunked-prefill expert product, %d-position chunk" % M,
                  "config 3: %d-token chunk, top-8 Zipf(1.1), %d-bit g64 experts (%s scales), x~N(0,1) bf16%s"
                  % (M, bits, args.scale_dtype, "" if as_bf16 else " values handed over as fp32"),
                  int(uniq * es), ms, args, {"flops_per_step": flops, "x_dtype": args.x_dtype})
    out["dtype"] = "bf16" if as_bf16 else "f32"
    out["roofline"] = {"bound": "hbm", "kernel": "fm_pf_rows (gate/up + down launches of one chunk)",
                       "achieved": round(uniq * es / (ev * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                       "frac": round(uniq * es / (ev * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                       "bytes_per_launch": int(uniq * es), "us_per_launch": round(ev * 1e3, 2),
                       "mfma_frac_of_bf16_peak": round(flops / (ev * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
    return out


def run_copy_probe(args):
    """Plain device copy of known size (1 GiB read + 1 GiB written per step): the
    calibration run for the FETCH_SIZE / WRITE_SIZE counters."""
    import torch
    dev = torch.device("cuda:0")
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device=dev).random_(0, 256)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        dst.copy_(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        dst.copy_(src)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    return _finish({}, "device copy GB/s (read + write)", "copy probe: 1 GiB uint8 torch copy_ per step",
                   2 * n, ms, args)


def run_stream_probe(args):
    """The streaming ceiling: 2 GiB read once per step by the library's probe kernel (one
    workgroup of twelve waves per CU, LDS-direct 16-byte loads into rings of two slots, no arithmetic) —
    what the memory system delivers to a kernel built like the expert kernels.  The headline
    is the dense order (pattern 0); the other two orders are reported beside it."""
    import torch
    from finchmoe_amd import FinchHip
    dev = torch.device("cuda:0")
    n = int(os.environ.get("FINCH_PROBE_BYTES", 2 << 30))
    bufs = [torch.empty(n, dtype=torch.uint8, device=dev).random_(0, 256) for _ in range(2)]
    ctx = FinchHip(0)
    torch.cuda.synchronize()
    rates = {}
    # patterns 0..7 read with the non-temporal hint the decode kernels give their weight loads,
    # 8 + p is walk p with ordinary caching
    for pattern, name in ((9, "contiguous_share_per_workgroup_ordinary_caching"), (8, "dense_ordinary_caching"),
                          (1, "contiguous_share_per_workgroup"), (2, "contiguous_share_per_wave"),
                          (3, "groups_of_4_workgroups_interleaved"), (4, "groups_of_8_workgroups_interleaved"),
                          (5, "groups_of_8_workgroups_of_one_xcd_interleaved"),
                          (6, "contiguous_share_per_workgroup_neighbours_on_one_xcd"),
                          (7, "groups_of_4_workgroups_of_one_xcd_interleaved"), (0, "dense")):
        def step(t, pattern=pattern):
            ctx.stream_probe_dev(bufs[t & 1].data_ptr(), n, pattern)
        ms, ev = _timed(ctx, step, args)
        rates[name] = round(n / (ev * 1e-3) / 1e9, 1)
    ctx.close()
    res = {"event_ms_per_step": round(ev, 5), "GBps_by_pattern": rates,
           "roofline": {"bound": "hbm", "kernel": "fm_stream_probe_k<0, non-temporal> (dense order)", "achieved": rates["dense"],
                        "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(rates["dense"] / HBM_PEAK_GBS, 4),
                        "traffic": None, "bytes_per_launch": n, "us_per_launch": round(ev * 1e3, 2)}}
    return _finish(res, "streaming read GB/s of the probe kernel", "stream probe: %d bytes read once per step, "
                   "two buffers alternating" % n, n, ms, args)


def _held_back(args):
    """Workloads that must not touch the GPU (see main): the ones of the faulted run whose code
    path has never completed a run at this size on this tree.  (decode_layer, gdn, gguf and
    gguf_chunk below 32 positions were on this list too; their launches — same kernels, same
    shapes — have since passed in the GPU suite, and every access of theirs is proven in bounds on
    the host.)"""
    return (args.workload == "gdn_prefill"
            or (args.workload == "decode_step" and (args.bits != 3 or args.scale_dtype != "bf16")))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="decode_step")
    ap.add_argument("--layers", type=int, default=L)
    ap.add_argument("--bits", type=int, default=3, choices=(3, 4),
                    help="affine code width of the decode_step and prefill workloads")
    ap.add_argument("--scale-dtype", default="bf16", choices=("bf16", "fp16"),
                    help="type of the group scales and biases (decode_step and prefill workloads)")
    ap.add_argument("--chunk", type=int, default=512, help="positions per chunk (prefill workload)")
    ap.add_argument("--x-dtype", default="bf16", choices=("bf16", "f32"),
                    help="prefill workload: hand the activations over as bf16 bits (config 3) or as fp32")
    ap.add_argument("--ramp-seconds", type=float, default=0.5,
                    help="untimed busy period before the warmup steps (clock ramp)")
    ap.add_argument("--graph", action="store_true",
                    help="moe_layer workload: replay the token from a captured HIP graph")
    ap.add_argument("--prefill-experts", type=int, default=0,
                    help="prefill workload: route uniformly over the first N experts instead of Zipf over all "
                         "(profile buckets: all items full / all items small)")
    ap.add_argument("--lm-format", default="affine8", choices=("affine8", "q4k", "q6k"),
                    help="lm_head workload: 8-bit affine, or the GGUF block formats")
    ap.add_argument("--forms", default="", help="comma-separated overrides of the library's kernel choice for A/B "
                    "runs: plain-dense, plain-gguf (the non-streaming kernels), per-position (no dense GEMM, "
                    "no grouped GGUF products for chunks), three-launches (moe_layer: experts and tail apart)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the path has no multi-GPU part); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    # One process of a run over several workloads ended in a GPU memory fault whose cause has not
    # been shown.  A workload listed here does not start, whatever the environment says: the walk
    # of its kernels' address ranges on the host (tests/test_host_bounds.py) found them in bounds,
    # so no cause has been shown, and its code path has never completed a run at this size.
    if _held_back(args):
        print("bench.py: workload %r with these options is held back: it was part of a run that ended in "
              "an unexplained GPU memory fault, and it stays off the GPU until a cause has been shown on "
              "the host and fixed" % args.workload, file=sys.stderr)
        sys.exit(4)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; there is no CPU fallback", file=sys.stderr)
        sys.exit(3)
    runners = {"decode_step": run_decode_step, "decode_layer": run_decode_layer, "gdn": run_gdn,
               "gguf": run_gguf, "gguf_chunk": run_gguf, "prefill": run_prefill, "lm_head": run_lm_head, "layer_tail": run_layer_tail,
               "moe_layer": run_moe_layer, "gdn_prefill": run_gdn_prefill,
               "copy_probe": run_copy_probe, "stream_probe": run_stream_probe}
    if args.workload not in runners:
        print("bench.py: unknown workload %r (have: %s)" % (args.workload, ", ".join(runners)),
              file=sys.stderr)
        sys.exit(2)
    # the case by name before the GPU is touched: if a kernel faults, the box may take the
    # output files with it and only the end of stderr comes back
    print("bench.py: workload=%s chunk=%d bits=%d scale_dtype=%s x_dtype=%s steps=%d warmup=%d graph=%s"
          % (args.workload, args.chunk, args.bits, args.scale_dtype, args.x_dtype, args.steps, args.warmup,
             bool(args.graph)), file=sys.stderr, flush=True)
    args.forms = [f for f in args.forms.split(",") if f]
    if args.forms:
        from finchmoe_amd import binding as fb
        known = {"plain-dense": fb.FORM_PLAIN_DENSE, "plain-gguf": fb.FORM_PLAIN_GGUF,
                 "per-position": fb.FORM_NO_DENSE_GEMM | fb.FORM_NO_GGUF_GROUP, "three-launches": 0,
                 "gguf-phases": fb.FORM_GGUF_PHASES, "gguf-one-launch": fb.FORM_GGUF_ONE_LAUNCH}
        bad = [f for f in args.forms if f not in known]
        if bad:
            print("bench.py: unknown --forms %s (have: %s)" % (bad, ", ".join(known)), file=sys.stderr)
            sys.exit(2)
        flags = 0
        for f in args.forms:
            flags |= known[f]
        rc = fb.load().fm_set_kernel_forms(flags)
        assert rc == 0, rc
    res = runners[args.workload](args)
    if args.forms:
        res.setdefault("config", {})["kernel_forms"] = args.forms
    print(json.dumps(res))


if __name__ == "__main__":
    main()
