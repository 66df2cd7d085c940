"""Builds csrc/*.hip into libscmx.so (gfx950) next to this file.  `python build.py` or build.build()."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libscmx.so")
SOURCES = ["api.hip", "gemm.hip", "gemv.hip", "rowops.hip", "quantize.hip", "attn.hip", "attn_prefill.hip", "silu_table.hip"]
# packed FP32 instructions are kept off (they have misbehaved on this hardware pool); no FMA contraction, so the
# FP32 epilogues and norms round exactly like a plain IEEE evaluation
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt", "-Wno-unused-command-line-argument", "-fconstexpr-steps=400000000",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if p.returncode:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    return out


def _build_id():
    """Source revision for scmx_version(): the git commit of the tree (with "+" when files differ from it), or "unknown"
    outside a checkout."""
    try:
        root = os.path.dirname(HERE)
        rev = subprocess.run(["git", "-C", root, "rev-parse", "--short=12", "HEAD"], capture_output=True, text=True, timeout=20)
        if rev.returncode:
            return "unknown"
        dirty = subprocess.run(["git", "-C", root, "status", "--porcelain", "--untracked-files=no"], capture_output=True,
                               text=True, timeout=20).stdout.strip()
        return rev.stdout.strip() + ("+" if dirty else "")
    except Exception:
        return "unknown"


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]
    bid = ['-DSCMX_BUILD_ID="%s"' % _build_id()]
    cmds = [[hipcc, *FLAGS, *(bid if s == "api.hip" else []), "-c", os.path.join(CSRC, s), "-o", o]
            for s, o in zip(SOURCES, objs)]
    with ThreadPoolExecutor(4) as ex:
        for out in ex.map(_run, cmds):
            if verbose and out.strip():
                print(out)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


def build_host_check(driver, out=None):
    """The library's sources and a C++ driver of the C ABI as ONE executable whose HOST code is instrumented with
    AddressSanitizer and UBSan (device code is compiled as usual and never runs in this check): for machines without a
    GPU, where every entry point ends at its argument checks or at the failing launch.  Returns the executable's path."""
    hipcc = os.environ.get("HIPCC", "hipcc")
    objdir = os.path.join(HERE, "build", "host_check")
    os.makedirs(objdir, exist_ok=True)
    out = out or os.path.join(objdir, "boundary_check")
    san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host",
           "-fno-sanitize-recover=undefined", "-g", "-fno-omit-frame-pointer"]
    flags = [f for f in FLAGS if f != "-O3"] + ["-O1"]
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]
    cmds = [[hipcc, *flags, *san, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(SOURCES, objs)]
    dobj = os.path.join(objdir, "driver.o")
    cmds.append([hipcc, "-x", "hip", *flags, *san, "-c", driver, "-o", dobj])
    with ThreadPoolExecutor(4) as ex:
        list(ex.map(_run, cmds))
    _run([hipcc, "--offload-arch=gfx950", "-fsanitize=address", "-fsanitize=undefined", "-o", out, dobj, *objs])
    return out


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
