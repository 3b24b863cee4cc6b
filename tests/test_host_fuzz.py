"""Damaged weight files against the C readers (finchmoe_amd/host/finch_files.c), under the host
compiler's address and undefined-behaviour sanitizers.  The readers map files that somebody
else wrote (finchmoe/infer.m:727-786 reads the manifest, 1025-1247 the GGUF directory): whatever
the bytes, a reader either refuses the file or hands out tensors that lie inside the mapping.
tests/host_fuzz/fuzz_files_main.c opens every file of a directory, reads every accepted tensor
end to end and runs the upload paths against counting doubles; a sanitizer report aborts it.
Host code only: nothing here touches a GPU."""
import os
import shutil
import struct
import subprocess

import numpy as np
import pytest

from finchmoe_amd import formats as F
from tests.test_host_loaders import write_dense, write_gguf

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    if not shutil.which("gcc"):
        pytest.skip("no host compiler")
    out = str(tmp_path_factory.mktemp("fuzzbin") / "fuzz_files_main")
    cmd = ["gcc", "-O1", "-g", "-std=gnu99", "-fsanitize=address,undefined,float-cast-overflow,float-divide-by-zero", "-fno-sanitize-recover=all",
           "-static-libasan", "-fno-omit-frame-pointer", "-ffp-contract=off",
           "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "host_fuzz", "fuzz_files_main.c"),
           os.path.join(ROOT, "finchmoe_amd", "host", "finch_files.c"), "-lm", "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode and "static-libasan" in r.stderr:
        cmd.remove("-static-libasan")
        r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return out


def _run(driver, kind, d):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:exitcode=97",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1:exitcode=98")
    r = subprocess.run([driver, kind, str(d)], capture_output=True, text=True, timeout=600, env=env)
    last = [l for l in r.stdout.splitlines() if l.startswith("file ")][-1:]
    assert r.returncode == 0, "sanitizer report on %s\n%s" % (last, r.stderr[-3000:])
    summary = r.stdout.strip().splitlines()[-1]
    assert summary.startswith("done "), summary
    return dict(kv.split("=") for kv in summary.split()[1:])


def _mutations(rng, data, n, structural=()):
    """n damaged copies of data: bit flips, overwritten integers, truncations, insertions —
    and the targeted ones (field offsets whose values the reader trusts most)."""
    out = []
    for i in range(n):
        b = bytearray(data)
        kind = i % 6
        if kind == 0 and len(b):                                  # a few flipped bits
            for _ in range(int(rng.integers(1, 4))):
                p = int(rng.integers(0, len(b)))
                b[p] ^= 1 << int(rng.integers(0, 8))
        elif kind == 1 and len(b) >= 8:                           # a 64-bit field replaced
            p = int(rng.integers(0, len(b) - 7))
            vals = [0, 1, 2**31, 2**32 - 1, 2**63, 2**64 - 1, len(b), len(b) + 1]
            v = vals[int(rng.integers(0, len(vals)))]
            b[p:p + 8] = struct.pack("<Q", v)
        elif kind == 2:                                           # cut short
            b = b[:int(rng.integers(0, max(1, len(b))))]
        elif kind == 3 and len(b):                                # random bytes over a span
            p = int(rng.integers(0, len(b)))
            m = int(rng.integers(1, 24))
            b[p:p + m] = bytes(rng.integers(0, 256, m, dtype=np.uint8))
        elif kind == 4:                                           # bytes inserted
            p = int(rng.integers(0, len(b) + 1))
            b[p:p] = bytes(rng.integers(0, 256, int(rng.integers(1, 16)), dtype=np.uint8))
        elif structural:
            p, width = structural[int(rng.integers(0, len(structural)))]
            vals = [0, 1, 255, 2**16, 2**31 - 1, 2**31, 2**32 - 1, 2**62, 2**64 - 1]
            v = vals[int(rng.integers(0, len(vals)))]
            b[p:p + width] = struct.pack("<Q", v)[:width]
        out.append(bytes(b))
    return out


def _gguf_bytes(tmp_path, rng):
    E, H, I = 3, 256, 256
    tensors = []
    for l in (0, 2):
        g, u, d = F.synth_gguf_layer(rng, E, H, I)
        tensors += [("blk.%d.ffn_gate_exps.weight" % l, 12, (H, I, E), g.tobytes()),
                    ("blk.%d.ffn_up_exps.weight" % l, 12, (H, I, E), u.tobytes()),
                    ("blk.%d.ffn_down_exps.weight" % l, 14, (I, H, E), d.tobytes())]
    tensors.append(("token_embd.weight", 0, (8, 4), np.arange(32, dtype=np.float32).tobytes()))
    kv = [("general.architecture", 8, "qwen3moe"), ("general.alignment", 4, 64),
          ("some.array", 9, (5, [1, -2, 3])), ("some.strings", 9, (8, ["a", "bc"])), ("x.f", 6, 1.5)]
    p = tmp_path / "base.gguf"
    write_gguf(str(p), kv, tensors, alignment=64)
    return p.read_bytes()


def test_gguf_reader_survives_damaged_files(driver, tmp_path):
    rng = np.random.default_rng(20261)
    base = _gguf_bytes(tmp_path, rng)
    head = base.index(b"blk.0.ffn_gate_exps.weight") - 8
    # header counts, the first tensor's name length, its dims, type and offset
    structural = [(8, 8), (16, 8), (head, 8), (head + 8 + 26, 4), (head + 8 + 26 + 4, 8),
                  (head + 8 + 26 + 4 + 24, 4), (head + 8 + 26 + 4 + 28, 8)]
    d = tmp_path / "gguf"
    d.mkdir()
    (d / "good.gguf").write_bytes(base)
    # the directory is what is under attack: damage its bytes, keep the (large) data behind it
    dir_len = head + 2048
    for i, m in enumerate(_mutations(rng, base[:dir_len], 360, structural)):
        (d / ("m%03d.gguf" % i)).write_bytes(m + base[dir_len:] if i % 6 != 2 else m)
    try:
        res = _run(driver, "gguf", d)
    finally:
        shutil.rmtree(d, ignore_errors=True)       # a few hundred MB of damaged copies
    assert int(res["files"]) == 361 and int(res["accepted"]) >= 1


def test_manifest_reader_survives_damaged_files(driver, tmp_path):
    rng = np.random.default_rng(20262)
    tensors = {}
    for name, (od, idim, bits) in {"a.weight": (8, 128, 4), "b.c.weight": (4, 256, 8), "d.weight": (16, 64, 3)}.items():
        _, W, S, B = F.synth_affine_tensor(rng, od, idim, bits)
        W32 = np.frombuffer(W.tobytes(), np.uint32).reshape(od, -1)
        tensors[name] = ("q", W32, S, B, bits, 64)
    tensors["norm.weight"] = ("bf16", F.bf16_trunc(rng.standard_normal(64).astype(np.float32)))
    pb, pj = tmp_path / "base.bin", tmp_path / "base.json"
    write_dense(str(pb), str(pj), tensors)
    js, blob = pj.read_bytes(), pb.read_bytes()
    d = tmp_path / "dense"
    d.mkdir()
    (d / "good.json").write_bytes(js)
    (d / "good.bin").write_bytes(blob)
    muts = _mutations(rng, js, 300)
    # and the numbers the reader trusts: offsets, sizes, shapes, bits pushed out of range
    import re
    nums = [m.span() for m in re.finditer(rb"\d+", js)]
    for k in range(120):
        a, b = nums[int(rng.integers(0, len(nums)))]
        vals = [0, 1, 7, 2**31, 2**32, 2**63, 2**64, 10**30, len(blob), len(blob) + 1]
        v = str(vals[int(rng.integers(0, len(vals)))]).encode()
        if k % 5 == 0:
            v = b"-" + v
        muts.append(js[:a] + v + js[b:])
    for i, m in enumerate(muts):
        (d / ("m%03d.json" % i)).write_bytes(m)
        # mostly the intact data file; sometimes a shortened or an empty one
        (d / ("m%03d.bin" % i)).write_bytes(blob if i % 7 else blob[:int(rng.integers(0, len(blob)))])
    try:
        res = _run(driver, "dense", d)
    finally:
        shutil.rmtree(d, ignore_errors=True)
    assert int(res["files"]) == len(muts) + 1 and int(res["accepted"]) >= 1


def test_quantizer_on_non_finite_and_extreme_weights(driver, tmp_path):
    """NaN, infinities, the largest floats and constant groups through the C quantizer under
    the sanitizers (float-to-integer conversions included): every call returns and packs."""
    env = dict(os.environ, UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1:exitcode=98")
    r = subprocess.run([driver, "quant", "-"], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0, r.stderr[-3000:]
    assert r.stdout.strip().endswith(tuple("0123456789")) and "accepted=8000" in r.stdout


def test_host_layer_bookkeeping_under_sanitizers(tmp_path):
    """finch_ops.c (the table from host weight pointers to resident tensors, the batch wrapper,
    the error paths) compiled with tests/host_fuzz/ops_table_main.c around it: doubles of the C
    ABI count registrations and releases; 60000 keys, reused pointers, failing registrations."""
    if not shutil.which("gcc"):
        pytest.skip("no host compiler")
    out = str(tmp_path / "ops_table_main")
    cmd = ["gcc", "-O1", "-g", "-std=gnu99", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           "-static-libasan", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "host_fuzz", "ops_table_main.c"), "-lm", "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode and "static-libasan" in r.stderr:
        cmd.remove("-static-libasan")
        r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    r = subprocess.run([out], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip().splitlines()[-1].startswith("done "), \
        (r.stdout[-500:], r.stderr[-2000:])
