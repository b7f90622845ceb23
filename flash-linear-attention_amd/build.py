"""Build libfla_hip.so (gfx950) from csrc/*.hip with hipcc, in-tree.

    python flash-linear-attention_amd/build.py [--force] [-j N]

Each translation unit is compiled to an object file under ``build/`` (kept out
of version control) and the objects are linked into ``fla_amd/lib/libfla_hip.so``.
hipcc cross-compiles, so this runs without a GPU.
"""
import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "fla_amd", "lib")
LIB_PATH = os.path.join(LIB_DIR, "libfla_hip.so")

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    # packed fp32 VALU forms are kept off
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# Keeps MFMA accumulators in ordinary vector registers: elementwise work on them (decay, scaling,
# conversion for stores) then needs no copies out of and back into the accumulation registers.
# Only where it measured faster (gdr_bwd_dhu 216 -> 204 us, gla_bwd_dh 166 -> 162 us); the forward state
# scans lose with it.
VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]
VGPR_FORM_SOURCES = {"gdr_bwd.hip", "gla_bwd.hip"}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _newest_header():
    hdrs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hdrs.append(os.path.join(HERE, "..", "include", "fla_hip.h"))
    return max(os.path.getmtime(h) for h in hdrs)


def _compile(src, force):
    obj = os.path.join(OBJ_DIR, src[:-4] + ".o")
    path = os.path.join(CSRC, src)
    if (not force and os.path.exists(obj)
            and os.path.getmtime(obj) >= max(os.path.getmtime(path), _newest_header())):
        return obj, ""
    cmd = [HIPCC] + FLAGS + (VGPR_FORM if src in VGPR_FORM_SOURCES else []) + ["-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{log}")
    return obj, log


def build(force=False, jobs=None, verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(lambda s: _compile(s, force), sources()))
    objs = [o for o, _ in results]
    for _, log in results:
        if log.strip() and verbose:
            print(log)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print(f"built {LIB_PATH} from {len(objs)} objects")
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", type=int, default=None)
    a = ap.parse_args()
    try:
        build(force=a.force, jobs=a.j)
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
