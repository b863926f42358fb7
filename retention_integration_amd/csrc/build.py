"""Builds libpower_retention_hip.so for gfx950 from the .hip sources in this directory.

    python retention_integration_amd/csrc/build.py [--jobs N]

The library is written next to the package (retention_integration_amd/libpower_retention_hip.so).
"""
import argparse
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(os.path.dirname(HERE), "libpower_retention_hip.so")
SOURCES = ["capi", "discumsum", "sympow_tn", "sympow_nn", "sympow_grad", "sympow_dvdk", "attention_fwd", "attention_bwd",
           "elementwise",
           "chunk_glue", "chunk_fwd", "chunk_bwd_dq", "decode", "cache"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

# Scheduling options per source file, kept where a whole training step at the headline shape measured faster with them
# than with the compiler's default strategy (same machine, alternating processes, clock settled): the memory-clause
# strategy takes 13 us off attention_bwd_dkv and 3 us off sympow_grad, the AMDGPU register-pressure trackers 4 us off
# sympow_tn.  The other strategies and files measured equal or slower (the forward attention kernel by 20-25 us
# under max-ilp and max-memory-clause).
FILE_FLAGS = {
    "attention_bwd": ["-mllvm", "-amdgpu-sched-strategy=max-memory-clause"],
    "chunk_bwd_dq": ["-mllvm", "-amdgpu-sched-strategy=max-memory-clause"],
    "sympow_grad": ["-mllvm", "-amdgpu-sched-strategy=max-memory-clause"],
    "sympow_dvdk": ["-mllvm", "-amdgpu-sched-strategy=max-memory-clause"],
    "sympow_tn": ["-mllvm", "-amdgpu-use-amdgpu-trackers=1"],
}


# headers beyond common.h and kernels.h that a source includes
FILE_HEADERS = {
    "sympow_nn": ["sympow_nn_dev.h"],
    "sympow_grad": ["sympow_grad_dev.h"],
    "sympow_dvdk": ["sympow_nn_dev.h", "sympow_grad_dev.h"],
}


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def stale(name):
    """Whether the object of a source is older than the source or a shared header."""
    obj = os.path.join(HERE, "build", name + ".o")
    if not os.path.exists(obj):
        return True
    deps = [os.path.join(HERE, name + ".hip"), os.path.join(HERE, "common.h"), os.path.join(HERE, "kernels.h")]
    deps += [os.path.join(HERE, h) for h in FILE_HEADERS.get(name, [])]
    return any(os.path.getmtime(d) > os.path.getmtime(obj) for d in deps)


def compile_one(name):
    obj = os.path.join(HERE, "build", name + ".o")
    extra = os.environ.get("PR_HIPCC_EXTRA_FLAGS", "").split()
    cmd = [hipcc(), *FLAGS, *FILE_FLAGS.get(name, []), *extra, "-c", os.path.join(HERE, name + ".hip"), "-o", obj]
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in p.stderr.splitlines() if "not a recognized feature" not in l)
    if p.returncode != 0:
        raise RuntimeError(f"hipcc failed for {name}.hip:\n{err}")
    return obj


def build(jobs=8, verbose=True, only_stale=False):
    """Compiles every source (only_stale: just those whose object is out of date) and links the library."""
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    todo = [n for n in SOURCES if not only_stale or stale(n)]
    if verbose and only_stale:
        print("compiling", todo)
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(compile_one, todo))
    objs = [os.path.join(HERE, "build", n + ".o") for n in SOURCES]
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objs]
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        raise RuntimeError("link failed:\n" + p.stderr)
    if verbose:
        print("built", OUT)
    return OUT


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=min(8, os.cpu_count() or 1))
    ap.add_argument("--changed", action="store_true", help="compile only the sources that changed since their object")
    args = ap.parse_args()
    build(args.jobs, only_stale=args.changed)
