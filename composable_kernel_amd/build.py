"""Builds libckx.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m composable_kernel_amd.build [--force]

Flags: -ffp-contract=off keeps the requant epilogue's fp32 multiplies unfused;
packed fp32 VALU forms are disabled for the device pass.

Three guards protect the kernels' hand-managed waits (the MFMA fragment reads of gemm_tile.hpp, conv_patch.hpp and
conv_pointwise.hpp are inline-assembly LDS reads that the compiler does not count in lgkmcnt; the kernels wait for
them themselves, so no compiler-made copy or spill of such a register may run before that wait):
  * every kernel's register report (-Rpass-analysis=kernel-resource-usage) is read, and the build FAILS if one of
    those kernels spills vector registers (the fused two-GEMM kernel, which reads LDS through compiler-known
    builtins, is allowed its four spilled registers in the long-sequence softmax variant);
  * the four-wave GEMM body (gemm_w4.hpp) also issues its MFMAs and direct loads as inline assembly: its kernels must
    use no scratch memory and exactly the AccVGPRs the source ties accumulators to (a compiler that moved an
    accumulator or fragment through another register between the assembly and its wait would show up there);
  * the compiler version the kernels were validated with is recorded below; another one FAILS the build unless
    CKX_ALLOW_UNVALIDATED_COMPILER=1 is set (then it builds with a loud warning; the bit-exact integer-operand GPU
    tests are the gate for adding a compiler to the list).
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
                "-Rpass-analysis=kernel-resource-usage", "-Wno-unused-command-line-argument"]
# hipcc --version lines of the toolchain whose code generation the GPU suite has validated
VALIDATED_COMPILERS = ("AMD clang version 22.0.0git (https://github.com/RadeonOpenCompute/llvm-project roc-7.2.0 26014 "
                       "7b800a19466229b8479a78de19143dc33c3ab9b5)",)


def compiler_version():
    r = subprocess.run([HIPCC, "--version"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    for line in r.stdout.splitlines():
        if "clang version" in line:
            return line.strip()
    return r.stdout.strip()[:200]


def check_compiler():
    import warnings
    v = compiler_version()
    if v not in VALIDATED_COMPILERS and os.environ.get("CKX_ALLOW_UNVALIDATED_COMPILER") != "1":
        raise RuntimeError(f"libckx: hipcc is {v!r}; its hand-waited inline-assembly kernels were validated with "
                           f"{VALIDATED_COMPILERS[0]!r}. Set CKX_ALLOW_UNVALIDATED_COMPILER=1 to build anyway, then run "
                           "the GPU suite (bit-exact integer-operand tests) before trusting the build.")
    if v not in VALIDATED_COMPILERS:
        warnings.warn(f"libckx is being built with an unvalidated compiler ({v}); its kernels wait for inline-assembly "
                      "LDS reads by hand and were validated with " + VALIDATED_COMPILERS[0] + ": run the GPU suite "
                      "(bit-exact integer-operand tests) before trusting this build", RuntimeWarning, stacklevel=2)
    return v


# kernels whose LDS fragment reads are inline assembly waited for by hand (mangled-name fragments)
HAND_WAITED_KERNELS = ("gemm_tile_kernel", "gemm_w4_kernel", "gemm_astream_kernel", "conv_patch_kernel", "conv_patch_wide_kernel",
                       "conv_pointwise_kernel")


def vgpr_spills(compiler_output):
    """(kernel, spilled VGPRs) for every hand-waited kernel of a -Rpass-analysis=kernel-resource-usage report that
    spills vector registers."""
    bad, name = [], "?"
    for line in compiler_output.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:", 1)[1].split("[", 1)[0].strip()
        elif "VGPRs Spill:" in line:
            n = int(line.split("VGPRs Spill:", 1)[1].split("[", 1)[0])
            if n and any(k in name for k in HAND_WAITED_KERNELS):
                bad.append((name, n))
    return bad


def scratch_users(compiler_output):
    """(kernel, bytes per lane) for every hand-waited kernel of the resource-usage report that uses scratch memory at
    all: spills, but also a per-lane array that the compiler could not keep in registers (the 3-D im2col kernels once
    held their window offsets there: scratch loads in every K iteration, and the compiler's waits for them, which wait
    for the prefetched K tiles as well)."""
    bad, name = [], "?"
    for line in compiler_output.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:", 1)[1].split("[", 1)[0].strip()
        elif "ScratchSize [bytes/lane]:" in line:
            n = int(line.split("ScratchSize [bytes/lane]:", 1)[1].split("[", 1)[0])
            if n and any(k in name for k in HAND_WAITED_KERNELS):
                bad.append((name, n))
    return bad


# gemm_w4_kernel: AccVGPRs a lane's accumulators are tied to (the last fragment row's live in VGPRs); the variants with
# D operands may park a few more values there
W4_AGPRS = 224
W4_AGPRS_FUSED_MAX = 232


def w4_register_faults(compiler_output):
    """(kernel, what) for every gemm_w4_kernel of the resource-usage report that uses scratch memory or another number of
    AccVGPRs than the source ties."""
    bad, name = [], None
    for line in compiler_output.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:", 1)[1].split("[", 1)[0].strip()
            name = name if "gemm_w4_kernel" in name else None
        elif name and "ScratchSize [bytes/lane]:" in line:
            n = int(line.split("ScratchSize [bytes/lane]:", 1)[1].split("[", 1)[0])
            if n:
                bad.append((name, f"{n} bytes of scratch per lane"))
        elif name and "AGPRs:" in line:
            n = int(line.split("AGPRs:", 1)[1].split("[", 1)[0])
            fused = "ILi1ELb1E" in name      # <DT_F16, FUSED = true, ...>
            if (n != W4_AGPRS and not fused) or (fused and not W4_AGPRS <= n <= W4_AGPRS_FUSED_MAX):
                bad.append((name, f"{n} AccVGPRs"))
    return bad


# conv_patch_kernel: the AccVGPRs hold exactly the wave's 36 weight fragments
PATCH_AGPRS = 144


def patch_register_faults(compiler_output):
    """(kernel, what) for every conv_patch_kernel of the resource-usage report that uses scratch memory or does not keep
    its weights -- and nothing else -- in AccVGPRs."""
    bad, name = [], None
    for line in compiler_output.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:", 1)[1].split("[", 1)[0].strip()
            name = name if "conv_patch_kernel" in name or "conv_patch_wide_kernel" in name else None
        elif name and "ScratchSize [bytes/lane]:" in line:
            n = int(line.split("ScratchSize [bytes/lane]:", 1)[1].split("[", 1)[0])
            if n:
                bad.append((name, f"{n} bytes of scratch per lane"))
        elif name and "AGPRs:" in line:
            n = int(line.split("AGPRs:", 1)[1].split("[", 1)[0])
            # (the 128-channel kernel: 60 of the 72 fp16 fragments, all 36 int8 ones)
            want = PATCH_AGPRS if "conv_patch_kernel" in name else (144 if "kernelILi0E" in name else 240)
            if n != want:
                bad.append((name, f"{n} AccVGPRs"))
    return bad


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

    check_compiler()

    def run(cmd):
        if verbose:
            print(" ".join(cmd))
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        lines = [l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l]
        # the register report: keep it out of the log, fail on vector register spills
        spills = vgpr_spills(r.stdout)
        scratch = scratch_users(r.stdout)
        w4_bad = w4_register_faults(r.stdout)
        patch_bad = patch_register_faults(r.stdout)
        out, skip = [], 0
        for l in lines:
            if "[-Rpass-analysis=kernel-resource-usage]" in l:
                skip = 2          # the remark is followed by a source line and a caret line
                continue
            if skip and (l.lstrip().startswith("|") or l.strip()[:1].isdigit() or l.startswith("In file included")):
                skip -= 1
                continue
            out.append(l)
        out = "\n".join(l for l in out if not l.startswith("In file included from") and "remarks generated" not in l)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed:\n" + "\n".join(lines))
        if spills:
            raise RuntimeError("vector register spills (the hand-managed LDS read waits do not survive them): "
                               + ", ".join(f"{k}: {n}" for k, n in spills))
        if scratch:
            raise RuntimeError("scratch memory in a kernel whose loads are counted by hand: "
                               + ", ".join(f"{k}: {n} bytes per lane" for k, n in scratch))
        if w4_bad:
            raise RuntimeError("four-wave GEMM body: register allocation differs from what its inline assembly assumes: "
                               + ", ".join(f"{k}: {what}" for k, what in w4_bad))
        if patch_bad:
            raise RuntimeError("input-patch conv kernel: register allocation differs from what its inline assembly assumes: "
                               + ", ".join(f"{k}: {what}" for k, what in patch_bad))
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
