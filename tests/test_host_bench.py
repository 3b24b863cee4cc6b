"""bench.py's contract where no GPU is needed: one GPU only, no CPU fallback, the routing
generator of the benchmark (distinct experts per layer, weights summing to one, Zipf skew)."""
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True,
                          text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_no_gpu_means_no_result():
    import torch
    if torch.cuda.is_available():
        return
    r = _run("--steps", "1", "--warmup", "0", "--no-cpu")
    assert r.returncode != 0 and "no CPU fallback" in r.stderr and r.stdout.strip() == ""


def test_unknown_workload_is_refused():
    import torch
    if not torch.cuda.is_available():
        return      # the GPU check comes first
    r = _run("--workload", "nonsense")
    assert r.returncode != 0 and "unknown workload" in r.stderr


def test_zipf_routing_of_the_benchmark():
    sys.path.insert(0, ROOT)
    from bench import zipf_routing
    idx, w = zipf_routing(np.random.default_rng(7), 64, 3, 256, 8)
    assert idx.shape == (64, 3, 8) and w.shape == (64, 3, 8)
    assert idx.min() >= 0 and idx.max() < 256
    for t in range(64):
        for l in range(3):
            assert len(set(idx[t, l].tolist())) == 8          # distinct per (token, layer)
    assert np.allclose(w.sum(-1), 1.0, atol=1e-6) and (w > 0).all()
    # skewed: the most frequent expert of a layer is hit far more often than the uniform 8/256
    for l in range(3):
        counts = np.bincount(idx[:, l].reshape(-1), minlength=256)
        assert counts.max() > 0.5 * 64
    # a fresh permutation per layer: the hot experts differ between layers
    hot = [int(np.bincount(idx[:, l].reshape(-1), minlength=256).argmax()) for l in range(3)]
    assert len(set(hot)) > 1


def test_cpu_baseline_legs_on_a_small_store():
    """bench.py's CPU leg on a store of 2 layers x 8 experts held in host memory: the port
    (oracle) leg, and — where oracle/_ref has been built — the leg through the reference's own
    compiled functions, which must reproduce the port's result bit for bit."""
    import numpy as np
    import torch
    import bench
    from finchmoe_amd import formats
    from oracle import oracle
    rng = np.random.default_rng(3)
    lo = formats.expert_layout(bench.H, bench.I, 3)
    Ls, E = 2, 8
    blob = torch.from_numpy(np.stack([formats.synth_expert_layer(rng, E, bench.H, bench.I, 3).reshape(E, -1)
                                      for _ in range(Ls)]))
    idx = np.stack([[rng.permutation(E) for _ in range(Ls)] for _ in range(3)]).astype(np.int32)
    w = rng.random((3, Ls, E)).astype(np.float32)
    x = rng.standard_normal((Ls, bench.H)).astype(np.float32)
    res = bench.cpu_baseline_decode(blob, lo, idx, w, x, budget_s=0.05, bits=3)
    assert res["unit"] == "GB/s" and res["cores"] == 1 and res["value"] > 0 and "sample" in res
    if oracle.ref_lib() is not None:
        assert res["kind"] == "reference" and res["equals_port_bit_for_bit"] is True
        assert res["port"]["value"] > 0
    else:
        assert res["kind"] == "port"
    # FP16 scales: the reference's files hold none, the port leg stands alone
    res16 = bench.cpu_baseline_decode(blob, lo, idx, w, x, budget_s=0.05, bits=3, scale_dtype=1)
    assert res16["kind"] == "port"


def test_cpu_baseline_of_the_dense_and_gguf_workloads():
    """The CPU legs of configs 1 and 4 on small operands held in host memory: same keys as the
    decode leg, the reference build when it is there, and the value the oracle computes."""
    import torch
    import bench
    from oracle import oracle
    rng = np.random.default_rng(5)
    out_dim, in_dim = 64, 256
    W = torch.from_numpy(rng.integers(0, 256, out_dim * in_dim // 2, dtype=np.uint8))
    S = torch.from_numpy((rng.random(out_dim * (in_dim // 64)).astype(np.float32).view(np.uint32) >> 16).astype(np.int16))
    B = torch.from_numpy((-rng.random(out_dim * (in_dim // 64)).astype(np.float32).view(np.uint32) >> 16).astype(np.int16))
    x = rng.standard_normal(in_dim).astype(np.float32)
    res = bench.cpu_baseline_dense([[(W, S, B, out_dim, in_dim, 4, 0)]], [x], budget_s=0.02, what="test tensor")
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in res
    assert res["cores"] == 1 and res["value"] > 0
    assert res["kind"] == ("reference" if oracle.ref_lib() is not None else "port")
    # GGUF: two layers of 8 experts in the benchmark's shapes, random blocks with small fp16 d
    def slab(nblocks, bsz, d_off, n_d):
        t = rng.integers(0, 256, (nblocks, bsz), dtype=np.uint8)
        d = (np.abs(rng.standard_normal((nblocks, n_d))) * 0.002).astype(np.float16)
        t[:, d_off:d_off + 2 * n_d] = d.view(np.uint8)
        return torch.from_numpy(t)
    E = 8
    gb, db = bench.I * (bench.H // 256), bench.H * (bench.I // 256)
    layers = [(slab(E * gb, 144, 0, 2), slab(E * gb, 144, 0, 2), slab(E * db, 210, 208, 1)) for _ in range(2)]
    idx = np.stack([[rng.permutation(E)[:4] for _ in range(2)] for _ in range(2)]).astype(np.int32)
    w = rng.random((2, 2, 4)).astype(np.float32)
    xs = rng.standard_normal((2, bench.H)).astype(np.float32)
    res = bench.cpu_baseline_gguf(layers, idx, w, xs, gb * 144, db * 210, budget_s=0.02)
    assert res["cores"] == 1 and res["value"] > 0 and res["unit"] == "GB/s" and "sample" in res
    # the roofline helper
    r = bench._roofline_hbm("k", 8e9, 1000.0, 2)
    assert r["bound"] == "hbm" and abs(r["achieved"] - 8000.0) < 1e-6 and abs(r["frac"] - 1.0) < 1e-9
    assert r["traffic"] is None and r["launches_per_step"] == 2


def test_every_workload_emits_roofline_and_cpu_baseline():
    """Without a GPU the workloads cannot run; their source must still build both objects: every
    runner of bench.py names a roofline, and every configuration of the benchmark (decode step,
    one layer, GDN projections, prefill, GGUF step and chunk) a cpu_baseline."""
    import ast
    import bench
    src = open(os.path.join(ROOT, "bench.py")).read()
    tree = ast.parse(src)
    funcs = {f.name: ast.get_source_segment(src, f) for f in tree.body if isinstance(f, ast.FunctionDef)}
    for name in ("run_decode_step", "run_decode_layer", "run_gdn", "run_gguf", "run_prefill", "run_lm_head",
                 "run_layer_tail", "run_moe_layer", "run_gdn_prefill", "run_stream_probe"):
        assert '"roofline"' in funcs[name], name
    for name in ("run_decode_step", "run_decode_layer", "run_gdn", "run_gguf", "run_prefill", "run_lm_head"):
        assert '"cpu_baseline"' in funcs[name], name
    assert funcs["run_gguf"].count('"cpu_baseline"') == 2       # the step and the chunk variant
    assert bench.HBM_PEAK_GBS == 8000.0 and bench.MFMA_BF16_PEAK_TFLOPS == 2500.0


def test_workloads_of_the_unexplained_fault_are_held_back():
    """Workloads that were part of the run that ended in an unexplained GPU fault do not start,
    whatever the environment says; the default workload and the chunked prefill are not among
    them."""
    env = dict(os.environ, FINCH_BENCH_UNVERIFIED="1")     # the former override no longer exists
    for extra in (["--workload", "gdn_prefill"], ["--bits", "4"], ["--scale-dtype", "fp16"]):
        r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--no-cpu", *extra], capture_output=True,
                           text=True, timeout=300, env=env)
        assert r.returncode == 4 and "held back" in r.stderr and r.stdout.strip() == "", extra
    import torch
    if not torch.cuda.is_available():
        for extra in ([], ["--workload", "prefill"], ["--workload", "gguf_chunk", "--chunk", "512"], ["--workload", "gdn"],
                      ["--workload", "gguf"], ["--workload", "decode_layer"], ["--workload", "gguf_chunk", "--chunk", "8"]):
            r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--no-cpu", *extra],
                               capture_output=True, text=True, timeout=300, env=env)
            assert r.returncode == 3, extra          # past the gate: stopped by the missing GPU
