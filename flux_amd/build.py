"""Build the native parts of flux_amd in-tree for gfx950.

  libfluxmi_kernels.so   HIP kernels + C-ABI (include/fluxmi.h)       <- flux_amd/csrc/kernels/*.hip
  flux_ths_pybind*.so    C++ torch extension with Flux's op surface    <- flux_amd/csrc/ths_op/*.cc

Usage: python -m flux_amd.build [--kernels-only] [--no-force]
Everything is rebuilt unless --no-force is given; with it, only translation units older than a file they
include are compiled again.  Outputs land in flux_amd/lib/ and travel with the source tree; nothing is installed.
"""
import argparse
import concurrent.futures
import hashlib
import os
import subprocess
import sys
import sysconfig

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "flux_amd")
KERNEL_DIR = os.path.join(PKG, "csrc", "kernels")
THS_DIR = os.path.join(PKG, "csrc", "ths_op")
LIB_DIR = os.path.join(PKG, "lib")
OBJ_DIR = os.path.join(PKG, "lib", "obj")
INCLUDE = os.path.join(ROOT, "include")

ARCH = "gfx950"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops is switched off on purpose: the compiler must not form v_pk_*_f32 by itself.
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", f"-I{INCLUDE}",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

# Per-file additions.  The block-scaled GEMM promotes every MFMA result with vector-ALU instructions right away:
# its MFMAs must write vector registers (the compiler's default for a kernel that uses both register files is
# the accumulation registers, which costs a v_accvgpr_read per element and promotion).
EXTRA_HIP_FLAGS = {"grouped_gemm_fp8_blockscale.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}

KERNEL_LIB = os.path.join(LIB_DIR, "libfluxmi_kernels.so")


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _newer(target, sources):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources)


def _deps_of(depfile):
    """Prerequisites listed in a make-style dependency file written by the compiler (-MD -MF)."""
    try:
        text = open(depfile).read()
    except OSError:
        return None
    text = text.replace("\\\n", " ")
    _, _, rhs = text.partition(":")
    return [t for t in rhs.split() if t]


def _object_current(obj, depfile, cmd):
    """True when `obj` was built by exactly `cmd` (recorded beside the dependency file) and is newer than everything
    it includes: a changed compiler flag rebuilds like a changed source does."""
    deps = _deps_of(depfile)
    if deps is None or not os.path.exists(obj):
        return False
    try:
        if open(depfile + ".cmd").read() != _cmd_stamp(cmd):
            return False
    except OSError:
        return False
    t = os.path.getmtime(obj)
    return all(os.path.exists(d) and os.path.getmtime(d) <= t for d in deps)


def _cmd_stamp(cmd):
    return hashlib.sha256("\0".join(cmd).encode()).hexdigest()


def build_kernels(force=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sorted(f for f in os.listdir(KERNEL_DIR) if f.endswith(".hip"))
    rebuilt = []

    def compile_one(name):
        obj = os.path.join(OBJ_DIR, name[:-4] + ".o")
        dep = obj[:-2] + ".d"
        cmd = [HIPCC, *HIP_FLAGS, *EXTRA_HIP_FLAGS.get(name, []), "-MD", "-MF", dep, "-c", os.path.join(KERNEL_DIR, name), "-o", obj]
        if not force and _object_current(obj, dep, cmd):
            return obj
        if os.path.exists(dep + ".cmd"):
            os.remove(dep + ".cmd")
        _run(cmd)
        with open(dep + ".cmd", "w") as f:
            f.write(_cmd_stamp(cmd))
        rebuilt.append(name)
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(compile_one, srcs))
    # Relink whenever an object is newer than the library (also after a link that failed: the stale library is
    # removed first, so a failed link never leaves an old one behind).
    if rebuilt or not os.path.exists(KERNEL_LIB) or any(os.path.getmtime(o) > os.path.getmtime(KERNEL_LIB) for o in objs):
        if os.path.exists(KERNEL_LIB):
            os.remove(KERNEL_LIB)
        _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", KERNEL_LIB])
    return KERNEL_LIB


def ths_ext_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(LIB_DIR, "flux_ths_pybind" + suffix)


def build_ths_op(force=True):
    """C++ host layer: Flux's torch-extension op surface over the C-ABI (no device code in it)."""
    import torch
    from torch.utils import cpp_extension

    srcs = sorted(os.path.join(THS_DIR, f) for f in os.listdir(THS_DIR) if f.endswith(".cc"))
    if not srcs:
        return None
    out = ths_ext_path()
    deps = srcs + [os.path.join(THS_DIR, f) for f in os.listdir(THS_DIR) if f.endswith(".h")]
    deps.append(os.path.join(INCLUDE, "fluxmi.h"))
    if not force and _newer(out, deps):
        return out
    os.makedirs(OBJ_DIR, exist_ok=True)
    inc = [f"-I{p}" for p in cpp_extension.include_paths()]
    inc += [f"-I{INCLUDE}", f"-I{sysconfig.get_paths()['include']}", "-I/opt/rocm/include"]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cxx11 = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    flags = [
        "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
        f"-D_GLIBCXX_USE_CXX11_ABI={cxx11}", "-DTORCH_EXTENSION_NAME=flux_ths_pybind",
        "-DTORCH_API_INCLUDE_EXTENSION_H", "-Wno-deprecated-declarations",
    ]

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, "ths_" + os.path.basename(src)[:-3] + ".o")
        _run(["g++", *flags, *inc, "-c", src, "-o", obj])
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(compile_one, srcs))
    _run([
        "g++", "-shared", *objs, "-o", out, f"-L{torch_lib}", f"-L{LIB_DIR}",
        "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python", "-lc10", "-lc10_hip", "-lfluxmi_kernels",
        "-L/opt/rocm/lib", "-lamdhip64",
        "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}",
    ])
    return out


CAPI_SMOKE = os.path.join(LIB_DIR, "capi_smoke")


def build_capi_smoke(force=True):
    """tests/capi_smoke.c: the C-ABI driven from plain C + the HIP runtime (no torch), linked against the library."""
    src = os.path.join(ROOT, "tests", "capi_smoke.c")
    if not os.path.exists(src):
        return None
    if not force and _newer(CAPI_SMOKE, [src, KERNEL_LIB, os.path.join(INCLUDE, "fluxmi.h")]):
        return CAPI_SMOKE
    _run(["gcc", "-O1", "-std=c11", "-ffp-contract=off", "-D__HIP_PLATFORM_AMD__=1", "-I/opt/rocm/include",
          f"-I{INCLUDE}", src, "-o", CAPI_SMOKE, f"-L{LIB_DIR}", "-lfluxmi_kernels", "-L/opt/rocm/lib", "-lamdhip64",
          "-lm", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"])
    return CAPI_SMOKE


def build_all(force=True, kernels_only=False):
    libs = [build_kernels(force)]
    if not kernels_only:
        ext = build_ths_op(force)
        if ext:
            libs.append(ext)
        smoke = build_capi_smoke(force)
        if smoke:
            libs.append(smoke)
    return libs


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--kernels-only", action="store_true")
    ap.add_argument("--no-force", action="store_true", help="skip targets newer than their sources")
    a = ap.parse_args()
    for lib in build_all(force=not a.no_force, kernels_only=a.kernels_only):
        print("built", os.path.relpath(lib, ROOT))
    sys.exit(0)
