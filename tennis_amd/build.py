"""Builds the gfx950 C-ABI library (libtsx_hip.so) in-tree with hipcc.

    python -m tennis_amd.build

Cross-compiles without a GPU.  The library is what the "hip" device operators, the
Python mirror of the operator API and every GPU test load; nothing is JIT-compiled.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libtsx_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: the fused epilogues must round exactly like the reference's chain of
# separate operators; fused multiply-adds are written explicitly where the reference has them.
# -packed-fp32-ops off: packed FP32 instructions are kept out of all device code.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    "-Rpass-analysis=kernel-resource-usage",
]


def scratch_users(compiler_output):
    """Kernels whose registers went to scratch memory, from hipcc's resource-usage remarks.

    A private array that is demoted to scratch turns every use into a memory round trip, which
    costs the MFMA kernels several-fold; the build refuses such an object file."""
    bad, name = [], None
    for line in compiler_output.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line:
            size = int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0].strip())
            if size and name:
                bad.append((name, size))
    return bad


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def build(verbose=True, jobs=8, incremental=False):
    """Compiles every kernel source and links the library.  incremental=True (development only) keeps an object
    file that is newer than its source and every header."""
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    procs = []
    objs = []
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".h"))]
    headers.append(os.path.join(ROOT, "include", "tsx_hip.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    for src in sources():
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header):
            continue
        cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        while sum(p.poll() is None for _, p in procs) >= jobs:
            procs[0][1].wait()
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        for name, size in scratch_users(out):
            print("FAILED: kernel %s uses %d bytes/lane of scratch" % (name, size), file=sys.stderr)
            failed = True
        # the host pass does not know the device-only feature flag; that note is harmless
        keep, skip = [], 0
        for l in out.splitlines():
            if "packed-fp32-ops" in l:
                continue
            if "remark:" in l:
                skip = 2      # the remark's source excerpt and caret line follow it
                while keep and keep[-1].startswith("In file included from"):
                    keep.pop()   # the include trail that led to the remark
                continue
            if skip and (" | " in l or l.strip().startswith("|")):
                skip -= 1
                continue
            skip = 0
            keep.append(l)
        out = "\n".join(keep)
        if out.strip() and verbose:
            print(out)
        if p.returncode != 0:
            print("FAILED:", src, file=sys.stderr)
            if not verbose:
                print(out, file=sys.stderr)
            failed = True
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    build_backend(verbose)
    return LIB_PATH


AIDS_LIB_PATH = os.path.join(LIB_DIR, "libtsx_hip_aids.so")


def build_aids(verbose=True, jobs=8):
    """The measurement build: the sources that carry phase stamps or probes compiled again with
    -DTSX_MEASUREMENT_AIDS, linked with the product's other objects into libtsx_hip_aids.so (bench.py --ceiling and
    the sustained-MFMA probe load it; nothing else does).  Needs a finished product build."""
    obj_dir = os.path.join(LIB_DIR, "obj")
    aids_dir = os.path.join(LIB_DIR, "obj_aids")
    os.makedirs(aids_dir, exist_ok=True)
    def carries_aids(src):
        text = open(src).read()
        if "TSX_MEASUREMENT_AIDS" in text:
            return True
        return any("TSX_MEASUREMENT_AIDS" in open(os.path.join(CSRC, h)).read()
                   for h in os.listdir(CSRC) if h.endswith(".hpp") and ('"%s"' % h) in text)
    procs, objs = [], []
    for src in sources():
        name = os.path.basename(src)[:-4] + ".o"
        if not carries_aids(src):
            objs.append(os.path.join(obj_dir, name))
            continue
        obj = os.path.join(aids_dir, name)
        objs.append(obj)
        cmd = [HIPCC] + [f for f in FLAGS if not f.startswith("-Rpass")] + ["-DTSX_MEASUREMENT_AIDS", "-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        while sum(p.poll() is None for _, p in procs) >= jobs:
            procs[0][1].wait()
    for src, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            print(out, file=sys.stderr)
            raise RuntimeError("hipcc failed: " + src)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", AIDS_LIB_PATH] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return AIDS_LIB_PATH


BACKEND_DIR = os.path.join(HERE, "backend")
BACKEND_LIB = os.path.join(LIB_DIR, "libtsx_backend.so")
BACKEND_SOURCES = ["ts/ts_api.cpp", "ts/base_ops.cpp", "hip/hip_device.cpp", "hip/hip_ops_quantized.cpp", "hip/hip_ops_float.cpp", "hip/hip_ops_glue.cpp", "hip/hip_ops_v2.cpp", "hip/hip_ops_fused.cpp", "capi_ops.cpp"]


def build_backend(verbose=True):
    """The C++ host side: TenniS-style operator classes for device "hip" over the C ABI (host code only;
    linked against libtsx_hip.so and the HIP runtime)."""
    cmd = [HIPCC, "-x", "c++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-D__HIP_PLATFORM_AMD__",
           "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include"]
    cmd += [os.path.join(BACKEND_DIR, s) for s in BACKEND_SOURCES]
    cmd += ["-o", BACKEND_LIB, "-L" + LIB_DIR, "-ltsx_hip", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN",
            "-Wl,-rpath,/opt/rocm/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return BACKEND_LIB


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv[1:])
    if "--aids" in sys.argv[1:]:
        build_aids()
