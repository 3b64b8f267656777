"""Builds libdwoconv1d_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libdwoconv1d_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # packed fp32 VALU forms are disabled for every device function in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # LDS reads keep their own 16-bit immediate offsets: merging them into ds_read2 forms
    # (8-bit offsets) costs one address add per pair in the unrolled tap gathers
    "-Xclang", "-target-feature", "-Xclang", "-load-store-opt",
    "-mllvm", "-amdgpu-load-store-vectorizer=0",
    "-Wno-unused-command-line-argument",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libdwoconv1d_hip.so cannot be built")
    return exe


PLANE_SHAPES = [(31, 56, 56), (31, 28, 28), (31, 14, 14), (31, 7, 7),
                (15, 56, 56), (15, 28, 28), (15, 14, 14), (15, 7, 7),
                (7, 56, 56), (7, 28, 28), (7, 14, 14),
                (31, 64, 64), (31, 32, 32), (31, 16, 16)]  # = DWO_PLANE_SHAPES
PLANE_TYPES = ["float", "bf16_t", "f16_t"]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass reports that it does not know the packed-fp32 feature: harmless
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l and "load-store-opt" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), err))
    if verbose and err.strip():
        print(err)


def build(verbose=False, jobs=None, only=None):
    """Compile csrc/dwo_api.hip and one csrc/dwo_inst.hip object per (element type, plane
    extent) in parallel, then link libdwoconv1d_hip.so into the package directory.  ``only``
    (substrings of object names, e.g. ``["dwo_api", "float_k31_56"]``) recompiles just those
    units and links them with the objects a previous full build left in place."""
    from concurrent.futures import ThreadPoolExecutor

    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    common = [hipcc()] + [f for f in HIPCC_FLAGS if f != "-shared"] + [
        "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-c"]
    units = [(os.path.join(CSRC, "dwo_api.hip"), os.path.join(objdir, "dwo_api.o"), [])]
    # longest translation units first (the register-plane extents, then the largest planes): the
    # build ends when the last worker does
    for K, H, W in sorted(PLANE_SHAPES, key=lambda s: (s[1] > 16, -s[0], -s[1] if s[1] > 16 else s[1])):
        for t in PLANE_TYPES:
            units.append((os.path.join(CSRC, "dwo_inst.hip"),
                          os.path.join(objdir, "dwo_inst_%s_k%d_%dx%d.o" % (t, K, H, W)),
                          ["-DDWO_INST_T=" + t, "-DDWO_INST_K=%d" % K, "-DDWO_INST_H=%d" % H,
                           "-DDWO_INST_W=%d" % W]))
    todo = units
    if only:
        todo = [u for u in units if any(tag in os.path.basename(u[1]) for tag in only)]
        missing = [u[1] for u in units if u not in todo and not os.path.exists(u[1])]
        if missing:
            raise RuntimeError("a partial build needs the objects of a full one; missing " + missing[0])
    jobs = jobs or min(len(todo), max(1, min(16, os.cpu_count() or 1)))
    with ThreadPoolExecutor(jobs) as pool:
        list(pool.map(lambda u: _run(common + u[2] + [u[0], "-o", u[1]], verbose), todo))
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC"] + [u[1] for u in units] +
         ["-o", LIB + ".tmp"], verbose)
    os.replace(LIB + ".tmp", LIB)
    return LIB


if __name__ == "__main__":
    import sys

    print(build(verbose="-q" not in sys.argv[1:], only=[a for a in sys.argv[1:] if a != "-q"] or None))
