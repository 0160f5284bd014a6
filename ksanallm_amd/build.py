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
    # one remark block per kernel with its registers, spills, scratch and LDS: read by check_resources below
    "-Rpass-analysis=kernel-resource-usage",
]

# The tile and streaming kernels issue their loads from inline assembly and count them by hand (`s_waitcnt vmcnt(N)`
# with a constant N); a register that an assembly load has been issued into must stay where it is until the wait that
# makes it valid.  A spill breaks that silently (the spilled copy is taken before the data has arrived), and scratch
# memory of any kind adds vector memory operations that the hand-kept counts do not know.  So the build refuses a
# kernel of these families that spills, uses scratch memory, or asks for more static LDS than a CU has.
GUARDED_KERNELS = ("_tile_kernel", "_splitk_kernel")
LDS_LIMIT = 160 * 1024


def parse_resource_remarks(text):
    """{kernel symbol: {"vgprs", "agprs", "sgprs", "scratch", "sgpr_spill", "vgpr_spill", "lds"}} from the compiler's
    kernel-resource-usage remarks."""
    import re
    keys = {"TotalSGPRs": "sgprs", "VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch",
            "SGPRs Spill": "sgpr_spill", "VGPRs Spill": "vgpr_spill", "LDS Size [bytes/block]": "lds"}
    out, cur = {}, None
    for line in text.splitlines():
        m = re.search(r"remark:\s+(.*?)\s*\[-Rpass-analysis=kernel-resource-usage\]", line)
        if not m:
            continue
        body = m.group(1)
        if body.startswith("Function Name:"):
            cur = out.setdefault(body.split(":", 1)[1].strip(), {})
        elif cur is not None and ":" in body:
            k, v = body.rsplit(":", 1)
            if k.strip() in keys and v.strip().lstrip("-").isdigit():
                cur[keys[k.strip()]] = int(v)
    return out


def check_resources(text, src=""):
    """Raises if a guarded kernel spills, uses scratch memory or exceeds the LDS; returns the parsed table."""
    table = parse_resource_remarks(text)
    bad = []
    for name, r in table.items():
        if not any(g in name for g in GUARDED_KERNELS):
            continue
        # (scalar registers spill into lanes of a vector register, not into memory: slower, not unsafe)
        if r.get("scratch", 0) or r.get("vgpr_spill", 0) or r.get("lds", 0) > LDS_LIMIT:
            bad.append("%s: scratch %d B/lane, VGPR spills %d, SGPR spills %d, LDS %d B" % (
                name, r.get("scratch", 0), r.get("vgpr_spill", 0), r.get("sgpr_spill", 0), r.get("lds", 0)))
    if bad:
        raise RuntimeError("kernels with hand-counted load pipelines must not spill or use scratch memory (%s):\n  %s"
                           % (src, "\n  ".join(bad)))
    return table


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(OBJ, src[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    check_resources(r.stderr, src)
    # the remarks (and the source lines the compiler quotes under them) are for the check, not for the reader
    if "warning:" not in err and "error:" not in err:
        return obj, ""
    return obj, "\n".join(l for l in err.splitlines() if "-Rpass-analysis=kernel-resource-usage" not in l)


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
