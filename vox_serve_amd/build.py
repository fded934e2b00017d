"""Build libvoxhip.so (gfx950) in-tree with hipcc.  Cross-compiles without a GPU."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libvoxhip.so")
SOURCES = ["core.hip", "kernels_lm.hip", "sampler.hip", "engine.hip", "codec.hip", "hybrid.hip"]
# the hybrid-mixer engine alone (context, sampler, its own kernels): what a process that only serves such a model has to compile
HYBRID_SOURCES = ["core.hip", "sampler.hip", "hybrid.hip"]
HYBRID_LIB = os.path.join(HERE, "libvoxhip_hybrid.so")
# -ffp-contract=off: the numeric contract spells every fused multiply-add as an explicit fmaf
# -packed-fp32-ops off: no packed fp32 instructions are generated from scalar float code (same results, instruction by instruction)
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-fPIC", "-Wno-unused-value",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"] + \
    os.environ.get("VOX_EXTRA_FLAGS", "").split()


def _hipcc():
    for c in ("/opt/rocm/bin/hipcc", "hipcc"):
        if os.path.isabs(c) and os.path.exists(c):
            return c
    return "hipcc"


def needs_build(lib: str = LIB) -> bool:
    if not os.path.exists(lib):
        return True
    t = os.path.getmtime(lib)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + [os.path.join(HERE, "..", "include", "voxhip.h")]
    return any(os.path.getmtime(d) > t for d in deps if os.path.exists(d))


def build(force: bool = False, verbose: bool = False, sources=None, lib: str = LIB) -> str:
    """Compile `sources` (default: all) and link them into `lib`.  Objects newer than their source and every header are kept."""
    if not force and not needs_build(lib):
        return lib
    srcs = [os.path.join(CSRC, s) for s in (sources or SOURCES) if os.path.exists(os.path.join(CSRC, s))]
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    hdrs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")] + [os.path.join(HERE, "..", "include", "voxhip.h"), __file__]
    newest_hdr = max(os.path.getmtime(h) for h in hdrs)
    for s in srcs:
        o = os.path.join(HERE, "build", os.path.basename(s) + ".o")
        objs.append(o)
        if not force and os.path.exists(o) and os.path.getmtime(o) > max(os.path.getmtime(s), newest_hdr):
            continue                    # this object is newer than its source and every header: keep it
        procs.append((s, subprocess.Popen([_hipcc(), *FLAGS, "-c", s, "-o", o], stdout=subprocess.PIPE,
                                          stderr=subprocess.STDOUT)))
    for s, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            sys.stderr.write(out.decode())
            raise RuntimeError(f"hipcc failed on {s}")
        if verbose and out:
            sys.stderr.write(out.decode())
    subprocess.check_call([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs])
    return lib


def build_hybrid(force: bool = False) -> str:
    """The reduced library for hybrid-mixer models (seconds to compile).  The full library contains it."""
    return build(force=force, sources=HYBRID_SOURCES, lib=HYBRID_LIB)


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
