"""Build ``libmedvision_hip.so`` for gfx950 with hipcc (``python -m medvision_amd.build``).

hipcc cross-compiles without a GPU.  Objects go to ``medvision_amd/lib/obj`` and the shared
library to ``medvision_amd/lib/libmedvision_hip.so`` (in-tree, not tracked by git).
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmedvision_hip.so")
# the same library with in-kernel time stamps in the tiled resampler (a measuring aid: `bench.py --timeline`)
TIMELINE_LIB_PATH = os.path.join(LIB_DIR, "libmedvision_hip_timeline.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
# per-file additions, keyed by source file name
FILE_FLAGS = {
    # matrix-core accumulators in ordinary vector registers: the kernel packs and stores them right
    # away, and copies between the two register classes would outnumber its arithmetic
    "roi_pool.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose=False, jobs=None):
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, os.path.basename(s)[:-4] + ".o") for s in sources]
    jobs = jobs or min(8, len(sources))
    with concurrent.futures.ThreadPoolExecutor(jobs) as pool:
        outs = list(pool.map(lambda so: _run([HIPCC, *FLAGS, *FILE_FLAGS.get(os.path.basename(so[0]), []),
                                              "-c", so[0], "-o", so[1]]),
                             zip(sources, objs)))
    link = _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs])
    # instrumented twin: only roi_resample.hip differs
    tl_src = os.path.join(CSRC, "roi_resample.hip")
    tl_obj = os.path.join(obj_dir, "roi_resample_timeline.o")
    outs.append(_run([HIPCC, *FLAGS, "-DMV_RESAMPLE_TIMELINE", "-c", tl_src, "-o", tl_obj]))
    tl_objs = [tl_obj if os.path.basename(o) == "roi_resample.o" else o for o in objs]
    link += _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", TIMELINE_LIB_PATH, *tl_objs])
    if verbose:
        for o in outs + [link]:
            if o.strip():
                print(o)
        print("built", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)
