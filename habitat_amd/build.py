"""Compile the HIP library for gfx950 with hipcc (in-tree, no JIT cache).

    python -m habitat_amd.build

writes habitat_amd/lib/libhabitat_mi.so.  hipcc cross-compiles, so no GPU is
needed to build.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libhabitat_mi.so")

SOURCES = ["api.hip", "host_records.hip", "wave_scale.hip", "mlp.hip", "trace.hip", "device_info.hip"]

# -packed-fp32-ops is switched OFF: the compiler must not form v_pk_*_f32.
HIPCC_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def sources():
    """Every file the library is compiled from (sources and headers)."""
    root = os.path.dirname(HERE)
    files = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC))
             if f.endswith((".hip", ".h"))]
    return files + [os.path.join(root, "include", "habitat_mi.h")]


def is_stale():
    """True when there is no library or a source file is newer than it."""
    if not os.path.exists(LIB_PATH):
        return True
    built = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(f) > built for f in sources() if os.path.exists(f))


def build(verbose=False):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", tmp] + srcs
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass says it does not know the packed-fp32 feature: harmless.
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
