"""Host-side proof that the kernels' global-memory accesses stay inside their buffers.

tests/host_bounds/bounds_main.cpp includes finchmoe_amd/csrc/fm_index.h — the header the kernels
take their share / unit / lane arithmetic from — and walks every (workgroup, unit, lane, load) of
the launches that bench.py and the GPU tests make, at their exact sizes (the 40 x 256 decode step
at 3 and 4 bits, one layer per call, the GatedDeltaNet projections for one and for 512 positions,
the vocabulary projection, the GGUF step — as three launches and as one — and chunk, the stream
probe), against the sizes of the
buffers those callers allocate; for the streaming kernels it also checks that the weights are read
exactly once.  Built with the address and undefined-behaviour sanitizers.  No GPU.
"""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "host_bounds", "bounds_main.cpp")


@pytest.fixture(scope="module")
def walker(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("bounds") / "bounds")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
                           "-fno-sanitize-recover=undefined", "-Wall", "-Werror", "-o", exe, SRC])
    return exe


def test_every_access_of_the_benchmark_launches_is_inside_its_buffer(walker):
    r = subprocess.run([walker], capture_output=True, text=True, timeout=900,
                       env=dict(os.environ, ASAN_OPTIONS="detect_leaks=0"))
    sys.stdout.write(r.stdout[-4000:])
    assert r.returncode == 0, r.stderr[-4000:]
    assert "all address ranges inside their buffers" in r.stdout
    # the launches the walk must have covered (a renamed or dropped case would otherwise go unseen)
    for case in ("stream_probe pattern 0", "gdn in_proj qkv+z 4-bit", "gdn out_proj 2048x4096",
                 "lm_head 248320x2048", "prefill dense 8192x2048 4-bit M=512",
                 "prefill dense 2048x4096 4-bit M=512", "prefill dense 2048x512 4-bit M=512",
                 "fused rows 40 groups x 8, 3-bit", "fused rows 40 groups x 8, 4-bit",
                 "fused rows 1 groups x 8, 3-bit", "split phases 40 groups x 8, 4-bit",
                 "fused (counters) 40 groups x 8, 4-bit", "gguf stream gate/up Q4_K 40 groups x 8",
                 "gguf stream down Q6_K 40 groups x 8", "gguf stream down Q6_K 8 groups x 8",
                 "fused rows, sweep of shapes", "fused rows + tail, LDS tables",
                 "gguf fused rows Q6_K down, 40 groups x 8, 2048x512", "gguf fused rows Q6_K down, 1 groups x 8, 2048x512",
                 "gguf fused rows Q4_K down, 3 groups x 8, 1024x512",
                 "chunk rows 512 positions x 8 on 256 experts, 3-bit, bf16 positions",
                 "chunk rows 512 positions x 8 on 256 experts, 4-bit, bf16 positions",
                 "chunk rows 2048 positions x 8 on 256 experts, 3-bit, bf16 positions",
                 "gguf chunk grouped 512 positions x 8 on 256 experts, 2048x512",
                 "gguf chunk grouped 36 positions x 4 on 12 experts, 4096x256"):
        assert ("ok  " + case) in r.stdout or ("ok  dense " + case) in r.stdout, case


def test_the_walk_notices_a_wrong_split(walker, tmp_path):
    """The same program with one index function broken on purpose (the first unit of a workgroup's
    second segment shifted by one: a gap, an overlap and a row step past the expert's last) must
    fail: a check that cannot fail proves nothing."""
    hdr = open(os.path.join(ROOT, "finchmoe_amd", "csrc", "fm_index.h")).read()
    needle = "p.first = lo - p.seg * segu;"
    assert needle in hdr
    bad_dir = tmp_path / "finchmoe_amd" / "csrc"
    bad_dir.mkdir(parents=True)
    (bad_dir / "fm_index.h").write_text(hdr.replace(needle, "p.first = lo - p.seg * segu + (qq == 1);"))
    tdir = tmp_path / "tests" / "host_bounds"
    tdir.mkdir(parents=True)
    (tdir / "bounds_main.cpp").write_text(open(SRC).read())
    exe = str(tmp_path / "bad")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-o", exe, str(tdir / "bounds_main.cpp")])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=900)
    assert r.returncode != 0 and "FAIL [fused rows" in r.stderr
