"""Compile the HIP sources under csrc/ into libscattermoe_amd.so (gfx950 only).

hipcc cross-compiles without a GPU, so this runs on any machine with ROCm.  The library is
placed inside the package directory and loaded from there by `_C`.
"""
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(PKG_DIR, "libscattermoe_amd.so")
# measurement aid of bench.py (csrc/bench/): a library of its own, so that the product library holds the MoE path only
PROBE_SRC = os.path.join(CSRC, "bench", "mfma_probe.hip")
PROBE_LIB_PATH = os.path.join(PKG_DIR, "libsmoe_bench_probe.so")

SOURCES = ["capi.hip", "route.hip", "group.hip", "s2s_generic.hip", "xty_generic.hip", "gemm_mfma.hip", "fused.hip", "router.hip", "s2s_rowdot.hip", "gemm_f32.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # keep the compiler from forming packed fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
]


def source_hash():
    """sha256 over every file the library is compiled from (csrc/*.hip, csrc/*.hpp, include/*.h), first 16 hex
    digits.  Baked into the library at build time; `_C.load` compares it with the sources it finds."""
    import hashlib
    inc = os.path.join(os.path.dirname(PKG_DIR), "include")
    files = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith((".hip", ".hpp"))]
    if os.path.isdir(inc):
        files += [os.path.join(inc, f) for f in sorted(os.listdir(inc)) if f.endswith(".h")]
    h = hashlib.sha256()
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the scattermoe_amd kernels need the ROCm toolchain to build")
    return exe


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), p.stdout))
    return p.stdout


def build(verbose=False, jobs=None):
    """Compile every source and link the shared library; always recompiles."""
    hipcc = _hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = [os.path.join(OBJ_DIR, s.replace(".hip", ".o")) for s in SOURCES]

    digest = source_hash()

    def one(pair):
        src, obj = pair
        extra = ['-DSMOE_SOURCE_HASH="%s"' % digest] if src == "capi.hip" else []
        out = _run([hipcc] + HIPCC_FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)

    jobs = jobs or min(len(SOURCES), max(1, (os.cpu_count() or 2)), 16)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(one, zip(SOURCES, objs)))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs)
    os.replace(tmp, LIB_PATH)
    if os.path.exists(PROBE_SRC):
        tmp = PROBE_LIB_PATH + ".tmp"
        _run([hipcc] + HIPCC_FLAGS + ["-shared", "-o", tmp, PROBE_SRC])
        os.replace(tmp, PROBE_LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
