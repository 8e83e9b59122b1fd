"""Build libhchip.so: gfx950 code objects via `hipcc --genco`, embedded into the host library.

Usage: python -m honeycrisp_amd.csrc.build   (or build_all() from Python)
Outputs, all in this directory: build/*.hsaco (intermediate) and libhchip.so.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
KERNEL_DIR = os.path.join(HERE, "kernels")
BUILD_DIR = os.path.join(HERE, "build")
LIB_PATH = os.environ.get("HCHIP_LIB_OUT", os.path.join(HERE, "libhchip.so"))
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# (code object, source, extra flags). -ffp-contract=off: the reference never fuses a*b+c.
# The packed-fp32 feature is switched off for every HIP compile.
KERNELS = [
    ("elementwise", "elementwise.hip", ["-ffp-contract=off"]),
    ("reduce", "reduce.hip", ["-ffp-contract=off"]),
    ("gather", "gather.hip", []),
    ("scan", "scan.hip", ["-ffp-contract=off"]),
    ("attention", "attention.hip", ["-ffp-contract=off"]),
    ("gemm", "gemm.hip", []),
    ("gemm_f16_fast", "gemm_f16_fast.hip", []),
    # (their epilogues can apply a bias / residual / GELU with the element-wise kernels' arithmetic)
    ("gemm_dma", "gemm_dma.hip", ["-ffp-contract=off"]),
    ("gemm_dma2", "gemm_dma2.hip", ["-ffp-contract=off"]),
    ("gemm_mi16", "gemm_mi16.hip", ["-ffp-contract=off"]),
    # the same three sources once more: kernels named *_m whose write-out applies the operations a
    # recording merged into the product (the plain kernels above contain none of that code)
    ("gemm_dma_m", "gemm_dma.hip", ["-ffp-contract=off", "-DHC_GEMM_MERGED=1"]),
    ("gemm_dma2_m_f16", "gemm_dma2.hip", ["-ffp-contract=off", "-DHC_GEMM_MERGED=1", "-DHC_GEMM_ONLY=16"]),
    ("gemm_dma2_m_f32", "gemm_dma2.hip", ["-ffp-contract=off", "-DHC_GEMM_MERGED=1", "-DHC_GEMM_ONLY=32"]),
    ("gemm_mi16_m", "gemm_mi16.hip", ["-ffp-contract=off", "-DHC_GEMM_MERGED=1"]),
]
DEVICE_FLAGS = [
    "--offload-arch=gfx950", "--genco", "-O3", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return proc.stdout


# Code objects whose kernels keep their accumulators in registers by construction: a kernel of these
# that needs private (scratch) memory has lost that property (a loop over the accumulators that the
# compiler no longer unrolls puts the whole array there and the kernel runs several times slower,
# with correct results), so the build refuses it. What is tolerated: a few registers, or one MFMA tile
# of 16 accumulators, parked once between the main loop and the write-out pass (the 256 x 256 tiles
# sit at the 256-VGPR limit; the edge kernels' write-out needs a few registers more): up to 96 bytes
# per lane in the plain kernels, up to 128 in the kernels with merged epilogues.
NO_SCRATCH = {"gemm_dma": 96, "gemm_dma2": 96, "gemm_mi16": 96, "gemm_f16_fast": 16,
              "gemm_dma_m": 128, "gemm_dma2_m_f16": 128, "gemm_dma2_m_f32": 128, "gemm_mi16_m": 128}


def kernels_with_scratch(remarks, allowed=0):
    """Names of kernels whose ScratchSize in -Rpass-analysis=kernel-resource-usage output exceeds
    `allowed` bytes per lane."""
    bad, current = [], None
    for line in remarks.splitlines():
        if "Function Name:" in line:
            current = line.split("Function Name:")[1].split()[0]
        elif "ScratchSize [bytes/lane]:" in line:
            size = int(line.split("ScratchSize [bytes/lane]:")[1].split()[0])
            if size > allowed:
                bad.append("%s (%d bytes/lane)" % (current, size))
    return bad


def kernels_with_promoted_private_data(remarks, granule=8192):
    """Names of kernels whose LDS size is not a whole number of `granule` bytes. The tiled GEMM
    kernels declare (BM + BN) * 256 bytes of LDS (the single-slice variants half of that), always a
    multiple of 8 KiB; anything on top is
    a private aggregate that the compiler moved into LDS (it does that with a struct or array whose
    member is picked at run time). Writing it there waits for every direct-to-LDS load in flight:
    one such 24-byte struct made a 2048 x 512 x 2048 product take 24 us instead of 9."""
    bad, current = [], None
    for line in remarks.splitlines():
        if "Function Name:" in line:
            current = line.split("Function Name:")[1].split()[0]
        elif "LDS Size [bytes/block]:" in line:
            size = int(line.split("LDS Size [bytes/block]:")[1].split()[0])
            if size % granule != 0:
                bad.append("%s (%d bytes of LDS)" % (current, size))
    return bad


def build_kernel(name, src, extra):
    out = os.path.join(BUILD_DIR, name + ".hsaco")
    # HCHIP_EXTRA_FLAGS: additional device-compile flags (kernel experiments, e.g. -DNAME=1)
    more = os.environ.get("HCHIP_EXTRA_FLAGS", "").split()
    check = ["-Rpass-analysis=kernel-resource-usage"] if name in NO_SCRATCH else []
    remarks = _run([HIPCC] + DEVICE_FLAGS + extra + more + check + ["-o", out, os.path.join(KERNEL_DIR, src)])
    bad = kernels_with_scratch(remarks, NO_SCRATCH[name]) if check else []
    if bad:
        os.remove(out)
        raise RuntimeError("%s: kernels that must not use scratch memory do: %s" % (src, ", ".join(bad)))
    bad = kernels_with_promoted_private_data(remarks) if check and name != "gemm_f16_fast" else []
    if bad:
        os.remove(out)
        raise RuntimeError("%s: private data was moved into LDS: %s" % (src, ", ".join(bad)))
    return out


def build_all(verbose=True):
    os.makedirs(BUILD_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=8) as pool:
        futures = [pool.submit(build_kernel, *k) for k in KERNELS]
        for f in futures:
            path = f.result()
            if verbose:
                print("built", os.path.relpath(path, HERE), os.path.getsize(path), "bytes")
    # The one source with device code linked into the library itself (a file-scope device array whose
    # address the host takes with hipGetSymbolAddress): compiled by hipcc to an object.
    noalloc_obj = os.path.join(BUILD_DIR, "noalloc.o")
    _run([HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-c",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          os.path.join(HERE, "noalloc.hip"), "-o", noalloc_obj])
    host_flags = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I" + os.path.join(ROCM, "include")]
    _run(["g++"] + host_flags + [
        "-Wa,-I," + BUILD_DIR,
        os.path.join(HERE, "hchip.cpp"), os.path.join(HERE, "embed.S"), noalloc_obj,
        "-o", LIB_PATH,
        "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(ROCM, "lib"),
        "-lpthread",
    ])
    if verbose:
        print("built", os.path.relpath(LIB_PATH, HERE), os.path.getsize(LIB_PATH), "bytes")
    if LIB_PATH == os.path.join(HERE, "libhchip.so"):
        # C++ host mirror + HCMatrixBench (links the library just built, and the Linux stand-in for
        # Accelerate that its CPU leg calls the way the reference's CPUBackend calls Accelerate)
        cpp = os.path.join(os.path.dirname(HERE), "cpp")
        bench = os.path.join(cpp, "HCMatrixBench")
        shim = os.path.join(os.path.dirname(os.path.dirname(HERE)), "swift", "honeycrisp-linux", "Sources", "Accelerate",
                            "accelerate_shim.c")
        shim_obj = os.path.join(BUILD_DIR, "accelerate_shim.o")
        _run(["gcc", "-O2", "-std=gnu11", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "-c", shim, "-o", shim_obj])
        _run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", os.path.join(cpp, "HCMatrixBench.cpp"), shim_obj, "-o", bench,
              "-L" + HERE, "-lhchip", "-Wl,-rpath,$ORIGIN/../csrc",
              "-L" + os.path.join(ROCM, "lib"), "-Wl,-rpath-link," + os.path.join(ROCM, "lib"), "-ldl", "-lm", "-lpthread"])
        if verbose:
            print("built", os.path.relpath(bench, HERE))
    return LIB_PATH


if __name__ == "__main__":
    build_all()
    sys.exit(0)
