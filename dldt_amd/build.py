"""Builds dldt_amd/libhipie.so (the C-ABI shared library) for gfx950 with hipcc.

Every translation unit under csrc/ is compiled to an object in csrc/build/ and linked into one
shared library next to this file.  Cross-compiles without a GPU.
"""
import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libhipie.so")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off",                       # float op order is part of the bit-exact contract
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes", "-Wno-pass-failed",
    "-I", os.path.join(os.path.dirname(HERE), "include"),
] + os.environ.get("HIPIE_EXTRA_FLAGS", "").split()


# per-file additions from the environment (HIPIE_BLOCK_FLAGS="-DHIPIE_BLOCK_STAMPS" builds the bottleneck-tail kernel,
# HIPIE_ATTENTION_FLAGS="-DHIPIE_ATT_STAMPS" the attention kernel, with cycle stamps; the library that ships is built without any)
EXTRA = {"conv_block.hip": os.environ.get("HIPIE_BLOCK_FLAGS", "").split(),
         "attention.hip": os.environ.get("HIPIE_ATTENTION_FLAGS", "").split()}


def _compile(src, force):
    obj = os.path.join(CSRC, "build", os.path.basename(src) + ".o")
    deps = [src] + glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(os.path.dirname(HERE), "include", "*.h"))
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) > os.path.getmtime(d) for d in deps):
        return obj
    cmd = [HIPCC] + FLAGS + EXTRA.get(os.path.basename(src), []) + (["-x", "hip"] if src.endswith(".hip") else []) + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force=True, jobs=8):
    os.makedirs(os.path.join(CSRC, "build"), exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))
    with concurrent.futures.ThreadPoolExecutor(jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs + ["-lpthread"]
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
