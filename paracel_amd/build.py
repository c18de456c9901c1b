"""Build steps for the native parts of the package (run on CPU; hipcc
cross-compiles gfx950 without a GPU).  Outputs land in-tree next to this file.
"""
import os
import shutil
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(_HERE)

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # keep packed-fp32 instructions out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
]


def _run(cmd, cwd=None):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True, cwd=cwd)


# The packed-fp32 switch is a device target feature; hipcc hands -Xclang options to
# its host pass as well (and -Xarch_device refuses options that take arguments), and the
# x86 backend answers with this line, once per function it compiles.  It says nothing
# about the code, so it is dropped from the output -- and only it: everything else the
# compiler prints still shows.
_HOST_PASS_NOISE = "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)"


def _run_hipcc(cmd):
    print("+", " ".join(cmd), flush=True)
    p = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
    rest = [ln for ln in p.stderr.splitlines() if ln.strip() != _HOST_PASS_NOISE]
    if rest:
        print("\n".join(rest), file=sys.stderr, flush=True)
    if p.returncode != 0:
        raise subprocess.CalledProcessError(p.returncode, cmd)


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def build_libplr():
    """HIP kernels + C ABI -> paracel_amd/libplr.so"""
    out = os.path.join(_HERE, "libplr.so")
    _run_hipcc([hipcc()] + HIPCC_FLAGS + ["-o", out, os.path.join(_HERE, "csrc", "plr_capi.hip")])
    return out


def build_libplr_gen():
    """Seeded shard generator (host C) -> paracel_amd/libplr_gen.so"""
    out = os.path.join(_HERE, "libplr_gen.so")
    _run(["gcc", "-O2", "-ffp-contract=off", "-fPIC", "-shared", "-pthread", "-Wall", "-Wextra",
          "-o", out, os.path.join(_HERE, "datagen", "plr_gen.c"), "-lm"])
    return out


def build_copy_probe():
    """Plain device copy of known size (counter calibration) -> paracel_amd/copy_probe"""
    out = os.path.join(_HERE, "copy_probe")
    flags = [f for f in HIPCC_FLAGS if f not in ("-fPIC", "-shared")]
    _run_hipcc([hipcc()] + flags + ["-o", out, os.path.join(_HERE, "csrc", "copy_probe.hip")])
    return out


def build_c_caller():
    """A plain-C99 caller of include/plr.h (gcc -std=c99 -pedantic -Wall -Werror), linked
    against libplr.so -> paracel_amd/plr_c_caller"""
    out = os.path.join(_HERE, "plr_c_caller")
    _run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-O2",
          "-I", os.path.join(ROOT, "include"), "-o", out,
          os.path.join(_HERE, "examples", "plr_c_caller.c"),
          "-L", _HERE, "-Wl,-rpath,$ORIGIN", "-lplr"])
    return out


def build_plan_check():
    """Host-only check of the width -> kernel-variant choice -> paracel_amd/plr_plan_check"""
    out = os.path.join(_HERE, "plr_plan_check")
    _run(["g++", "-O2", "-std=c++17", "-Wall", "-Wextra", "-o", out,
          os.path.join(_HERE, "csrc", "plr_plan_check.cpp")])
    return out


def build_worker():
    """Host side of the worker path (g++): parameter-server process, reducer
    plugin, GPU LR worker, shard tool ->
    paracel_amd/{plr_ps_server,liblr_update.so,plr_lr_worker,plr_ridge_worker,plr_shard_tool,
    plr_ps_roundtrip,plr_comm_check}"""
    _run(["make", "-B", "-C", os.path.join(_HERE, "worker")])
    return [os.path.join(_HERE, f) for f in ("plr_ps_server", "liblr_update.so", "plr_lr_worker",
                                             "plr_ridge_worker", "plr_shard_tool",
                                             "plr_ps_roundtrip", "plr_comm_check")]


def build_all():
    return [build_libplr(), build_libplr_gen(), build_copy_probe(), build_plan_check(),
            build_c_caller()] + build_worker()
