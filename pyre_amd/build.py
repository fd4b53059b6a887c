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


def build(verbose=True, jobs=8, extra_flags=(), out_dir=None, incremental=False, only=None):
    """out_dir (with extra_flags): a diagnostics variant of the library beside the product build, e.g. -DPYRE_PHASE_TS.
    incremental: sources whose object is newer than the source and every header are not compiled again (development
    aid; the default compiles everything).  only: compile just these source base names and link with the other objects."""
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    hdr_time = max(os.path.getmtime(h) for h in glob.glob(os.path.join(CSRC, "*.h")) + [os.path.join(CSRC, "..", "..", "include", "pyre_hip.h")])
    objs = []
    lib = LIB if out_dir is None else os.path.join(out_dir, "libpyre_hip.so")
    if out_dir is not None:
        os.makedirs(out_dir, exist_ok=True)
    todo = [(s, (s[:-4] + ".o") if out_dir is None else os.path.join(out_dir, os.path.basename(s)[:-4] + ".o"), tuple(extra_flags)) for s in srcs]
    def fresh(job):
        src, obj, _ = job
        if only is not None:
            return os.path.basename(src)[:-4] not in only and os.path.exists(obj)
        return incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), hdr_time)
    objs.extend(j[1] for j in todo if fresh(j))
    todo = [j for j in todo if not fresh(j)]
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
