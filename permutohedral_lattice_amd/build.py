"""Compile the HIP library for gfx950, in-tree.

    python permutohedral_lattice_amd/build.py

(run as a script: importing the package needs the library this file builds)

Produces ``permutohedral_lattice_amd/libpermutohedral_hip.so`` (cross-compiles without a GPU).
"""
import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_HERE)
LIB_PATH = os.path.join(_HERE, "libpermutohedral_hip.so")

SOURCES = [os.path.join(_HERE, "csrc", name)
           for name in ("pl_kernels.hip", "pl_kernels_f64.hip", "pl_order.hip", "pl_gather.hip", "pl_api.cpp")]

# -ffp-contract=off: the lattice's integer results need unfused IEEE float operations.
# -munsafe-fp-atomics: float atomicAdd becomes the hardware global_atomic_add_f32.
# packed-fp32 ops are switched off for the device code.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-I" + os.path.join(_ROOT, "include"), "-I" + os.path.join(_HERE, "csrc"),
]


def source_hash():
    """Short hash of the sources the library is built from (every .hip, .h and .cpp under csrc/
    but the command-line tool): the library reports it (pl_library_info), so that a measurement or
    a harness can tell which build of the kernels it is talking to."""
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(_HERE, "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h", ".cpp")) and not name.startswith("bilateral_filter_cli"):
            h.update(name.encode())
            h.update(open(os.path.join(csrc, name), "rb").read())
    return h.hexdigest()[:12]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def build(verbose=False):
    cmd = [hipcc()] + FLAGS + ["-DPL_SOURCE_HASH=0x%sLL" % source_hash()] + SOURCES + ["-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 target feature: harmless
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


CPP_DRIVER_SRC = os.path.join(_ROOT, "tests", "cpp", "compare_cpu_and_gpu.cpp")
CPP_DRIVER_BIN = os.path.join(_ROOT, "tests", "cpp", "compare_cpu_and_gpu.bin")


def build_cpp_driver(verbose=False):
    """The C++ CPU-vs-GPU comparison driver (tests/cpp), linked against the HIP library and the
    CPU oracle; both are found through rpath entries relative to the binary."""
    oracle_dir = os.path.join(_ROOT, "oracle")
    cmd = [hipcc(), "-O2", "-std=c++17", "-Wno-unused-command-line-argument",
           "-I" + os.path.join(_ROOT, "include"), "-I" + oracle_dir, CPP_DRIVER_SRC,
           "-L" + _HERE, "-lpermutohedral_hip", "-L" + oracle_dir, "-loracle",
           "-Wl,-rpath,$ORIGIN/../../permutohedral_lattice_amd", "-Wl,-rpath,$ORIGIN/../../oracle",
           "-o", CPP_DRIVER_BIN]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout)
    return CPP_DRIVER_BIN


CLI_SRC = os.path.join(_HERE, "csrc", "bilateral_filter_cli.cpp")
CLI_BIN = os.path.join(_HERE, "bilateral_filter_hip.bin")


def build_cli(verbose=False):
    """The command-line bilateral filter for BMP images (the reference's test_bilateral_gpu)."""
    cmd = [hipcc(), "-O2", "-std=c++17", "-Wno-unused-command-line-argument",
           "-I" + os.path.join(_ROOT, "include"), CLI_SRC, "-L" + _HERE, "-lpermutohedral_hip",
           "-Wl,-rpath,$ORIGIN", "-o", CLI_BIN]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout)
    return CLI_BIN


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_cli(verbose=True))
    sys.exit(0)
