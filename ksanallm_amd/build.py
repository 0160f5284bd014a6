"""Builds libksq_hip.so (gfx950) in-tree with hipcc.  `python -m ksanallm_amd.build`."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libksq_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    # packed-fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-ignored-attributes",
    # the assembly statements that write M0 say so in their clobber lists; the compiler answers that M0 is a reserved
    # register (it never keeps a value of its own there across a statement), once per instantiation
    "-Wno-inline-asm",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(OBJ, src[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(verbose=False, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(jobs) as ex:
        results = list(ex.map(_compile, sources()))
    objs = [o for o, _ in results]
    if verbose:
        for _, e in results:
            if e.strip():
                print(e, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


LAYERS = os.path.join(HERE, "layers")
LAYERS_LIB = os.path.join(HERE, "libksq_layers.so")
LAYER_TEST = os.path.join(ROOT, "tests", "cpp", "layer_test")


def build_layers():
    """C++ layer classes (host code only) -> libksq_layers.so, and the driver tests/cpp/layer_test that links them."""
    srcs = sorted(os.path.join(LAYERS, f) for f in os.listdir(LAYERS) if f.endswith(".cpp"))
    common = [HIPCC, "-std=c++17", "-O2", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + LAYERS,
              "-Wno-unused-command-line-argument"]
    link = ["-L" + HERE, "-lksq_hip", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(common + ["-shared", "-o", LAYERS_LIB] + srcs + link, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("layer build failed:\n" + r.stderr)
    r = subprocess.run(common + ["-o", LAYER_TEST, os.path.join(ROOT, "tests", "cpp", "layer_test.cpp"),
                                 "-L" + HERE, "-lksq_layers", "-lksq_hip",
                                 "-Wl,-rpath,$ORIGIN/../../ksanallm_amd"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("layer test build failed:\n" + r.stderr)
    return LAYERS_LIB, LAYER_TEST


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_layers())
