"""Builds pyre_amd/csrc/libpyre_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
import concurrent.futures
import glob
import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB = os.path.join(CSRC, "libpyre_hip.so")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(job):
    src, obj, extra = job
    cmd = ["hipcc", *FLAGS, *extra, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    return src, obj, r.returncode, (r.stdout + r.stderr)


def build(verbose=True, jobs=8, extra_flags=(), out_dir=None):
    """out_dir (with extra_flags): a diagnostics variant of the library beside the product build, e.g. -DPYRE_PHASE_TS."""
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = []
    lib = LIB if out_dir is None else os.path.join(out_dir, "libpyre_hip.so")
    if out_dir is not None:
        os.makedirs(out_dir, exist_ok=True)
    todo = [(s, (s[:-4] + ".o") if out_dir is None else os.path.join(out_dir, os.path.basename(s)[:-4] + ".o"), tuple(extra_flags)) for s in srcs]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, obj, rc, out in ex.map(_compile, todo):
            msg = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
            if verbose and msg:
                print(msg)
            if rc != 0:
                raise RuntimeError("hipcc failed on %s\n%s" % (src, out))
            objs.append(obj)
    r = subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed\n" + r.stdout + r.stderr)
    return lib


if __name__ == "__main__":
    print(build())
    sys.exit(0)
