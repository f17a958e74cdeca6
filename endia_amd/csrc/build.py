"""Build libendia_hip.so (gfx950 only) in-tree with hipcc.

    python endia_amd/csrc/build.py       # compile every csrc/*.hip, link endia_amd/libendia_hip.so

It is run as a script (or loaded by path), never through `import endia_amd`, because importing the
package requires the library this script produces.

The library has no dependency beyond the HIP runtime; nothing here needs a GPU.
"""
import concurrent.futures
import os
import subprocess
import sys

CSRC = os.path.dirname(os.path.abspath(__file__))
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(os.path.dirname(CSRC), "libendia_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 instructions are switched off for every device translation unit
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unused-command-line-argument",
] + os.environ.get("ENDIA_EXTRA_HIPCC_FLAGS", "").split()


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass says it does not know the packed-fp32 feature; that line is noise
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr))
    return obj, err


def build(verbose=True, jobs=None):
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), 8)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(jobs) as ex:
        for obj, err in ex.map(_compile, srcs):
            objs.append(obj)
            if verbose and err.strip():
                print(err, file=sys.stderr)
    tmp = LIB_PATH + ".tmp"
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build()
