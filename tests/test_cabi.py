"""The C-ABI library loads and exports every symbol include/finch_hip.h declares; argument
validation that needs no GPU.  No compute calls here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "finch_hip.h")).read()
    return sorted(set(re.findall(r"FM_API[^;(]*?\b(fm_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_surface():
    names = _declared()
    assert len(names) >= 35
    for must in ("fm_ctx_create", "fm_experts_upload_layer", "fm_moe_decode", "fm_moe_decode_step_dev",
                 "fm_moe_prefill", "fm_matvec_batch", "fm_matvec_prefill", "fm_gguf_moe_decode",
                 "fm_dequant_expert", "fm_gguf_dequant_expert"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from finchmoe_amd import binding
    L = binding.load()
    missing = [n for n in _declared() if not hasattr(L, n)]
    assert not missing, missing
    # the binding covers the whole header
    assert sorted(L._signatures) == _declared()


def test_host_library_exports_every_declared_symbol():
    """libfinchops.so: every function include/finch_ops.h and include/finch_files.h declare."""
    from finchmoe_amd import binding
    binding.load()
    L = C.CDLL(os.path.join(ROOT, "finchmoe_amd", "libfinchops.so"))
    names = []
    for h in ("finch_ops.h", "finch_files.h"):
        text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", h)).read(), flags=re.S)
        names += re.findall(r"^[a-z][A-Za-z0-9_ \*]*?\b([a-z][a-z0-9_]+)\s*\(", text, flags=re.M)
    assert len(names) >= 45 and "fast_batch_matvec" in names and "finch_ops_open_gguf" in names
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing


def test_status_strings():
    from finchmoe_amd import binding
    L = binding.load()
    for code in (0, -1, -2, -3, -4, -5):
        assert L.fm_status_string(code)
    assert L.fm_status_string(0) == b"ok"


def test_no_gpu_means_error_not_fallback():
    """Without a device the context cannot be created and nothing computes on the CPU."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from finchmoe_amd import FinchHip, FinchError
    with pytest.raises(FinchError):
        FinchHip(0)
    from finchmoe_amd import binding
    L = binding.load()
    assert L.fm_sync(None) == binding.ERR_ARG
    assert L.fm_moe_decode(None, 0, None, None, None, 8, None, None, 0) == binding.ERR_ARG


def test_product_does_not_import_oracle():
    """The package must not reach into oracle/ (the oracle is the checker, never the product)."""
    pkg = os.path.join(ROOT, "finchmoe_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".c", ".h", ".hip", ".cpp")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def test_integration_example_compiles_and_links(tmp_path):
    """examples/engine_moe_layer.c — the reference's call sites written against the two host
    headers — compiles as strict C99 and links against the built libraries; without a GPU it
    ends with the library's error, not a crash."""
    import shutil
    import subprocess
    if not shutil.which("gcc"):
        pytest.skip("no host compiler")
    libdir = os.path.join(ROOT, "finchmoe_amd")
    out = str(tmp_path / "engine_moe_layer")
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror",
                        "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "examples", "engine_moe_layer.c"),
                        "-L", libdir, "-lfinchops", "-lfinchhip", "-lm", "-Wl,-rpath," + libdir, "-o", out],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    import torch
    if not torch.cuda.is_available():
        r = subprocess.run([out, str(tmp_path)], capture_output=True, text=True, timeout=120)
        assert r.returncode == 1 and "finch_ops_init" in r.stderr
