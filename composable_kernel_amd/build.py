"""Builds libckx.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m composable_kernel_amd.build [--force]

Flags: -ffp-contract=off keeps the requant epilogue's fp32 multiplies unfused;
packed fp32 VALU forms are disabled for the device pass.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libckx.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-Wno-unused-command-line-argument"]


def sources():
    return [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC))]


def stale():
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    deps = sources() + [os.path.join(ROOT, "include", "ckx.h")]
    return any(os.path.getmtime(p) > t for p in deps)


def build_lib(force=False, verbose=False, extra_flags=()):
    """Compile csrc/*.hip (side by side) into objects and link lib/libckx.so. Returns the library path."""
    if not force and not stale():
        return LIB
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIBDIR, exist_ok=True)
    units = [f for f in sources() if f.endswith(".hip")]
    objs = [os.path.join(LIBDIR, os.path.basename(u)[:-4] + ".o") for u in units]

    def run(cmd):
        if verbose:
            print(" ".join(cmd))
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed:\n" + out)
        if verbose and out.strip():
            print(out)

    common = [HIPCC] + DEVICE_FLAGS + list(extra_flags) + ["-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    with ThreadPoolExecutor(max_workers=len(units)) as pool:
        list(pool.map(lambda uo: run(common + ["-c", uo[0], "-o", uo[1]]), zip(units, objs)))
    run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB])
    for o in objs:
        os.remove(o)
    return LIB


HOST = os.path.join(HERE, "host")
BINDIR = os.path.join(HERE, "bin")
HOST_PROGRAMS = {
    "ckx_profiler": os.path.join(HOST, "profiler", "ckx_profiler.cpp"),
    "example_gemm_requant_relu_requant_int8": os.path.join(HOST, "example", "gemm_requant_relu_requant_int8.cpp"),
}


def build_host(force=False, verbose=False):
    """Compile the C++ host programs (operator classes are header-only) against libckx.so."""
    build_lib()
    os.makedirs(BINDIR, exist_ok=True)
    hdrs = [os.path.join(HOST, "ckx", f) for f in os.listdir(os.path.join(HOST, "ckx"))] + [LIB]
    out = []
    for name, src in HOST_PROGRAMS.items():
        exe = os.path.join(BINDIR, name)
        out.append(exe)
        if not force and os.path.exists(exe) and all(os.path.getmtime(exe) >= os.path.getmtime(p) for p in hdrs + [src]):
            continue
        cmd = [HIPCC, "-x", "c++", "-std=c++17", "-O2", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
               "-I" + os.path.join(ROOT, "include"), "-I" + HOST, src, "-x", "none", "-o", exe,
               "-L" + LIBDIR, "-lckx", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN/../lib",
               "-Wl,-rpath,/opt/rocm/lib", "-Wno-unused-command-line-argument"]
        if verbose:
            print(" ".join(cmd))
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError("host build failed:\n" + r.stdout)
    return out


if __name__ == "__main__":
    print(build_host(force="--force" in sys.argv, verbose=True))
    print(build_lib(force="--force" in sys.argv, verbose=True))
