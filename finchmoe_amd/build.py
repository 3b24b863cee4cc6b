"""Build libfinchhip.so (HIP kernels + C ABI) for gfx950, in-tree.

    python -m finchmoe_amd.build            # build if sources are newer
    python -m finchmoe_amd.build --force
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libfinchhip.so")
HOSTLIB = os.path.join(HERE, "libfinchops.so")
SOURCES = ["fm_api.hip", "fm_decode.hip", "fm_dense.hip", "fm_dequant.hip", "fm_gguf.hip",
           "fm_prefill.hip", "fm_tail.hip", "fm_route.hip", "fm_probe.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops off: v_pk_*_f32 forms are not trusted on the target pool
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, verbose=False, extra_flags=(), lib=None):
    """extra_flags / lib: alternative builds (experiments) into another file."""
    global LIB
    if lib:
        LIB, force = lib, True
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)]
    deps.append(os.path.join(HERE, "..", "include", "finch_hip.h"))
    if force or _stale(LIB, deps):
        objs = []
        procs = []
        os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
        for src in SOURCES:
            obj = os.path.join(HERE, "build", ("alt_" if lib else "") + src.replace(".hip", ".o"))
            objs.append(obj)
            cmd = [HIPCC] + FLAGS + list(extra_flags) + ["-c", os.path.join(CSRC, src), "-o", obj]
            if verbose:
                print(" ".join(cmd))
            procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE,
                                                stderr=subprocess.STDOUT, text=True)))
        for src, p in procs:
            out, _ = p.communicate()
            out = "\n".join(l for l in out.splitlines()
                            if "packed-fp32-ops' is not a recognized feature" not in l)
            if p.returncode:
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
            if out.strip() and verbose:
                print(out)
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        subprocess.check_call(cmd)
    host = os.path.join(HERE, "host")
    host_src = [os.path.join(host, f) for f in ("finch_ops.c", "finch_files.c")]
    host_hdr = [os.path.join(HERE, "..", "include", f) for f in ("finch_hip.h", "finch_ops.h", "finch_files.h")]
    if not lib and (force or _stale(HOSTLIB, host_src + host_hdr)):
        # -ffp-contract=off: the quantizer reproduces fp32 array arithmetic operation by operation
        subprocess.check_call(["gcc", "-O2", "-std=c99", "-ffp-contract=off", "-fPIC", "-shared", "-Wall",
                               "-I", os.path.join(HERE, "..", "include"),
                               "-o", HOSTLIB] + host_src + ["-L", HERE, "-lfinchhip", "-lm",
                               "-Wl,-rpath,$ORIGIN"])
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
    print(LIB)
