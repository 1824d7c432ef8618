"""Compiles the gfx950 library and the C++ host layer in-tree with hipcc.

    python -m sapphire_amd.build            # everything
    python -m sapphire_amd.build hip host   # selected parts

Outputs (git-ignored, next to the package so that they travel with the tree):
    sapphire_amd/libsapphire_hip.so    C ABI of include/sapphire_hip.h
    sapphire_amd/libsapphire_host.so   C++ operator layer (Sapphire:: namespace)
    tests/host_harness/libhost_harness.so   C view of that layer for the Python tests
    sapphire_amd/libsapphire_probe.so  measurement aid for bench.py --only mfma_ceiling (not
                                       part of the C ABI, not loaded by anything else)
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
OBJ = os.path.join(ROOT, "build", "obj")

HIP_LIB = os.path.join(PKG, "libsapphire_hip.so")
HOST_LIB = os.path.join(PKG, "libsapphire_host.so")

ARCH = "gfx950"

# -packed-fp32-ops is switched off for every device compile: the compiler must
# not form packed fp32 instructions from ordinary float code on this target.
HIP_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-ignored-attributes",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the gfx950 library cannot be built")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(line for line in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in line)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _sources(folder, exts):
    return sorted(os.path.join(folder, f) for f in os.listdir(folder)
                  if os.path.splitext(f)[1] in exts)


def _compile_all(sources, flags, tag):
    os.makedirs(OBJ, exist_ok=True)
    hipcc = _hipcc()
    objs = []
    jobs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources) or 1)) as pool:
        for src in sources:
            obj = os.path.join(OBJ, tag + "_" + os.path.basename(src) + ".o")
            objs.append(obj)
            jobs.append(pool.submit(_run, [hipcc] + flags + ["-c", src, "-o", obj]))
        for job in jobs:
            text = job.result()
            if text.strip():
                print(text)
    return objs


def build_hip():
    """hipcc --offload-arch=gfx950 over every csrc/*.hip -> libsapphire_hip.so"""
    objs = _compile_all(_sources(CSRC, {".hip"}), HIP_FLAGS, "hip")
    _run([_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", HIP_LIB] + objs)
    return HIP_LIB


PROBE_DIR = os.path.join(PKG, "probe")
PROBE_LIB = os.path.join(PKG, "libsapphire_probe.so")


def build_probe():
    """The matrix-core ceiling probe behind `bench.py --only mfma_ceiling`."""
    objs = _compile_all(_sources(PROBE_DIR, {".hip"}), HIP_FLAGS, "probe")
    _run([_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", PROBE_LIB] + objs)
    return PROBE_LIB


def build_host():
    """C++17 operator layer, linked against the C ABI library beside it."""
    flags = ["-O2", "-std=c++17", "-fPIC", "-x", "c++",
             "-I" + os.path.join(ROOT, "include"), "-I" + HOST]
    objs = _compile_all(_sources(HOST, {".cpp"}), flags, "host")
    _run([_hipcc(), "-shared", "-fPIC", "-o", HOST_LIB] + objs +
         ["-L" + PKG, "-lsapphire_hip", "-Wl,-rpath,$ORIGIN"])
    return HOST_LIB


HARNESS_DIR = os.path.join(ROOT, "tests", "host_harness")
HARNESS_LIB = os.path.join(HARNESS_DIR, "libhost_harness.so")


def build_harness():
    """C entry points over the C++ layer for the Python parity tests."""
    flags = ["-O2", "-std=c++17", "-fPIC", "-x", "c++",
             "-I" + os.path.join(ROOT, "include"), "-I" + HOST, "-I" + CSRC]
    objs = _compile_all(_sources(HARNESS_DIR, {".cpp"}), flags, "harness")
    _run([_hipcc(), "-shared", "-fPIC", "-o", HARNESS_LIB] + objs +
         ["-L" + PKG, "-lsapphire_host", "-lsapphire_hip", "-Wl,-rpath,$ORIGIN/../../sapphire_amd"])
    return HARNESS_LIB


def build_oracle():
    """The CPU checker (test infrastructure): oracle/liboracle.so and, when the
    reference tree is present, oracle/_ref/libsapphire_ref.so."""
    _run(["make", "-B", "-C", os.path.join(ROOT, "oracle")])


def build_all():
    build_hip()
    build_probe()
    build_host()
    build_harness()
    build_oracle()


if __name__ == "__main__":
    parts = sys.argv[1:] or ["all"]
    for part in parts:
        {"hip": build_hip, "probe": build_probe, "host": build_host, "harness": build_harness,
         "oracle": build_oracle, "all": build_all}[part]()
        print("built", part)
