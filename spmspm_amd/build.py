"""Builds libSpMM_API.so for gfx950 in-tree (spmspm_amd/lib/)."""
import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
LIBPATH = os.path.join(LIBDIR, "libSpMM_API.so")

SOURCES = ["spmm_api.hip", "encoder_device.hip", "encoder.cpp"]
# Packed-fp32 VALU forms are switched off for every device compile.  Kernel arguments are preloaded into scalar
# registers when a wave starts (gfx950 supports it; a kernel then begins without the round trip for its argument
# block): 0.25-0.4 us per call on every shape measured, 3 % of a 5120x5120 call.
DEVICE_FLAGS = [
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared", "-fvisibility=default",
    *DEVICE_FLAGS,
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-Wno-inline-asm",  # the wide kernel's direct-to-LDS load names m0, which the compiler calls reserved
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the ROCm toolchain is required to build libSpMM_API.so")
    return exe


VARIANTS_LIBPATH = os.path.join(LIBDIR, "libSpMM_API_variants.so")


def build_library(verbose=False, extra_flags=(), out=None):
    """Compile every source into one shared library.  Always recompiles."""
    out = out or LIBPATH
    os.makedirs(LIBDIR, exist_ok=True)
    cmd = [hipcc(), *HIPCC_FLAGS, *extra_flags, "-I", os.path.join(ROOT, "include"), "-I", CSRC]
    cmd += [os.path.join(CSRC, s) for s in SOURCES]
    cmd += ["-o", out + ".tmp", "-lpthread"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building " + os.path.basename(out))
    if verbose and proc.stderr.strip():
        sys.stderr.write(proc.stderr)
    os.replace(out + ".tmp", out)
    return out


def build_variants_library(verbose=False):
    """The test build: the same library plus the two comparison kernels (-DSPMM_KEEP_VARIANTS) and the switch
    SpMM_Debug_SetKernelVariant that selects them.  Only tests load it."""
    return build_library(verbose=verbose, extra_flags=("-DSPMM_KEEP_VARIANTS",), out=VARIANTS_LIBPATH)


HARNESS_SRC = os.path.join(ROOT, "tests", "cpp", "harness.cpp")
HARNESS_PATH = os.path.join(LIBDIR, "spmm_harness")


def build_harness(verbose=False):
    """Compile the C++ caller (tests/cpp/harness.cpp) against the library: the reference harness's call sequence
    through the `__half*` encoder overload and the 14-argument entry point.  Run by the GPU tests."""
    cmd = [hipcc(), "-O2", "-std=c++17", "--offload-arch=gfx950", "-Wno-unused-command-line-argument",
           "-I", os.path.join(ROOT, "include"), HARNESS_SRC, "-L", LIBDIR, "-lSpMM_API",
           "-Wl,-rpath,$ORIGIN", "-o", HARNESS_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building the C++ harness")
    os.replace(HARNESS_PATH + ".tmp", HARNESS_PATH)
    return HARNESS_PATH


PROBE_SRC = os.path.join(CSRC, "stream_probe.hip")
PROBE_PATH = os.path.join(LIBDIR, "stream_probe")


def build_stream_probe(verbose=False):
    """The read-streaming probe (csrc/stream_probe.hip): a stand-alone program bench.py runs to put the machine's
    own read ceiling next to the data-sheet peak."""
    cmd = [hipcc(), "-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-unused-command-line-argument", PROBE_SRC, "-o", PROBE_PATH + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building the stream probe")
    os.replace(PROBE_PATH + ".tmp", PROBE_PATH)
    return PROBE_PATH


def kernel_resources(source, extra_flags=()):
    """Compiles the device side of one source to assembly and returns, per kernel, the registers it uses and what
    it spills: {mangled name: {"vgpr": n, "sgpr": n, "vgpr_spill": n, "sgpr_spill": n, "scratch_bytes": n}}.
    A kernel that spills inside its tile loop loses a large factor without failing any numerical test."""
    import re
    import tempfile
    fd, asm = tempfile.mkstemp(suffix=".s")
    os.close(fd)
    try:
        cmd = [hipcc(), "-O3", "-std=c++17", "--offload-arch=gfx950", *DEVICE_FLAGS,
               "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", *extra_flags,
               "-I", os.path.join(ROOT, "include"), "-I", CSRC, "--cuda-device-only", "-S",
               os.path.join(CSRC, source), "-o", asm]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            sys.stderr.write(proc.stdout + proc.stderr)
            raise RuntimeError("hipcc failed compiling " + source)
        text = open(asm).read()
    finally:
        os.unlink(asm)
    out = {}
    keys = {"vgpr_count": "vgpr", "sgpr_count": "sgpr", "vgpr_spill_count": "vgpr_spill",
            "sgpr_spill_count": "sgpr_spill", "private_segment_fixed_size": "scratch_bytes"}
    for block in text.split("  - .agpr_count")[1:]:  # one entry of amdhsa.kernels each
        name = re.search(r"^\s+\.name:\s+(\S+)", block, re.M)
        if not name:
            continue
        out[name.group(1)] = {v: int(re.search(r"^\s+\.%s:\s+(\d+)" % k, block, re.M).group(1))
                              for k, v in keys.items()}
    return out


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_variants_library(verbose=True))
    print(build_harness(verbose=True))
    print(build_stream_probe(verbose=True))
