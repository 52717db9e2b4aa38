"""Build the HIP libraries for gfx950 with hipcc.

Run as ``python -m tritonformer_amd._build`` (recompiles what changed; ``--force``
recompiles everything).  Every ``csrc/*.hip`` file is compiled to an object (in
parallel) and linked into ``libtritonformer_amd.so`` next to this file, where
``_lib.py`` loads it with ctypes; ``csrc/diag/*.hip`` become
``libtritonformer_amd_diag.so`` (diagnostics, never loaded by an operator).

The product library carries a hash of the sources it was built from
(``tf_source_hash``); ``_lib.load`` compares it with the sources next to it and
refuses a library that is older than they are.
"""
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
DIAG = os.path.join(CSRC, "diag")
INCLUDE = os.path.join(ROOT, "include")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libtritonformer_amd.so")
DIAG_LIB_PATH = os.path.join(HERE, "libtritonformer_amd_diag.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wno-unused-result",
    # packed-fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources(folder=CSRC):
    return sorted(f for f in os.listdir(folder) if f.endswith(".hip"))


def _headers():
    out = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith(".h")]
    out += [os.path.join(INCLUDE, f) for f in sorted(os.listdir(INCLUDE)) if f.endswith(".h")]
    return out


def source_hash():
    """sha256 over every file the product library is built from (names and contents)."""
    h = hashlib.sha256()
    for path in [os.path.join(CSRC, f) for f in sources()] + _headers():
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:32]


def _compile(job):
    folder, src, force, extra = job
    obj = os.path.join(OBJ_DIR, ("diag_" if folder == DIAG else "") + src[:-4] + ".o")
    path = os.path.join(folder, src)
    if not force and os.path.exists(obj):
        newest = max(os.path.getmtime(p) for p in [path, os.path.abspath(__file__)] + _headers())
        if os.path.getmtime(obj) > newest and not extra:
            return obj, ""
    cmd = [HIPCC, *FLAGS, *extra, "-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    return obj, err


def _link(objs, path):
    tmp = path + ".tmp"
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, path)


def build_library(verbose=True, jobs=None, force=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    diag = sources(DIAG)
    # api.hip holds the source hash: always recompiled (it is tiny)
    define = [f'-DTF_SOURCE_HASH="{source_hash()}"']
    todo = [(CSRC, s, force, define if s == "api.hip" else []) for s in srcs] + [(DIAG, s, force, []) for s in diag]
    jobs = jobs or min(len(todo), int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, todo))
    if verbose:
        for (_, err), job in zip(results, todo):
            if err.strip():
                print(f"[{job[1]}] {err}", file=sys.stderr)
    _link([o for o, _ in results[: len(srcs)]], LIB_PATH)
    _link([o for o, _ in results[len(srcs):]], DIAG_LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources, {DIAG_LIB_PATH} from {len(diag)}")
    return LIB_PATH


if __name__ == "__main__":
    build_library(force="--force" in sys.argv)
