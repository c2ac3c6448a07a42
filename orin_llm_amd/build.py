"""Builds liborin_fa.so (HIP kernels + C ABI + llm::cuda shim) for gfx950, in-tree, and beside it the two
measurement-aid libraries that bench.py and one GPU test load (liborin_fa_stamps.so, liborin_fa_bench.so)."""
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liborin_fa.so")
# The timeline build: the same sources, the two attention kernels and the matrix-vector kernel compiled with -DORIN_FA_STAMPS so that their
# stage marks store the wall clock.  A measurement aid for bench.py's timeline workloads; never the library that is timed.
STAMPS_LIB = os.path.join(HERE, "liborin_fa_stamps.so")
STAMPED = ("fa_prefill.hip", "fa_decode.hip", "gemv_mfma.hip", "fa_api.hip")
# Read-only stand-ins and a do-nothing kernel (csrc/bench_aids.hip), a library of their own: the product exports none of them.
BENCH_LIB = os.path.join(HERE, "liborin_fa_bench.so")
BENCH_SOURCE = os.path.join(HERE, "csrc", "bench_aids.hip")
# The cut-off builds: the decode split kernel with parts taken out (-DORIN_FA_DECODE_PROBE=flags, see fa_decode.hip;
# results wrong by design), one library per flag set, for bench.py's cut-off workloads.  Measurement aids, built
# only on request: build(probes=True), `python -m orin_llm_amd.build --probes`, or the cut-off workloads themselves.
PROBE_FLAGS = (1, 3, 7, 15, 31)
PROBE_LIB = os.path.join(HERE, "liborin_fa_probe_{}.so")
# ... and of the prefill kernel (-DORIN_FA_PREFILL_PROBE=flags, see fa_prefill.hip)
PPROBE_FLAGS = (1, 2, 4, 7, 8, 16, 32, 64)
PPROBE_LIB = os.path.join(HERE, "liborin_fa_pprobe_{}.so")
OBJ_DIR = os.path.join(HERE, "_obj")
SOURCES = [os.path.join(HERE, "csrc", n)
           for n in ("fa_prefill.hip", "fa_decode.hip", "kv_cache.hip", "rope.hip", "gemv.hip", "gemv_mfma.hip", "layer_ops.hip",
                     "layer_api.hip", "fa_api.hip", "llm_cuda_shim.cpp")]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-exceptions",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the leading scalar arguments of a kernel arrive in registers when a wave starts, instead of
    # behind a trip to memory (the attention kernels put what their first loads need there)
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
]
# Per source: the matrix-vector kernels' matrix instructions leave their sums in vector registers (the default puts
# them in accumulation registers, from which the vector ALU has to fetch each with a move before it can use it).
EXTRA_FLAGS = {"gemv_mfma.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


# The prefill kernel's hand-placed instruction stream (matrix-result and vector-write wait states counted by
# hand, registers of loads in flight) was validated against the code this compiler generates around it;
# another compiler may move what the counts rely on, so it is refused until the GPU tests have been re-run
# with it (set ORIN_FA_ALLOW_UNTESTED_TOOLCHAIN=1 to do exactly that).
TESTED_TOOLCHAINS = ("roc-7.2.0",)


def check_toolchain():
    out = subprocess.run([HIPCC, "--version"], capture_output=True, text=True).stdout
    if any(t in out for t in TESTED_TOOLCHAINS) or os.environ.get("ORIN_FA_ALLOW_UNTESTED_TOOLCHAIN") == "1":
        return
    raise RuntimeError("hipcc is not one of the toolchains the hand-scheduled kernels were validated with "
                       f"({', '.join(TESTED_TOOLCHAINS)}); re-run the GPU tests with ORIN_FA_ALLOW_UNTESTED_TOOLCHAIN=1 "
                       "before trusting this build.  hipcc --version:\n" + out)


def _run(cmd):
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
    return " ".join(cmd)


def build(verbose=False, probes=False):
    """Compiles every source (in parallel) and links the shared library and its timeline build.  Always recompiles.
    probes=True also builds the eleven cut-off libraries (measurement aids whose results are wrong by design)."""
    check_toolchain()
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = [os.path.join(OBJ_DIR, os.path.basename(s) + ".o") for s in SOURCES]
    cmds = [[HIPCC] + FLAGS + EXTRA_FLAGS.get(os.path.basename(s), []) + ["-c", s, "-o", o] for s, o in zip(SOURCES, objs)]
    stamped = {s: os.path.join(OBJ_DIR, os.path.basename(s) + ".stamps.o") for s in SOURCES if os.path.basename(s) in STAMPED}
    cmds += [[HIPCC] + FLAGS + EXTRA_FLAGS.get(os.path.basename(s), []) + ["-DORIN_FA_STAMPS", "-c", s, "-o", o] for s, o in stamped.items()]
    bench_obj = os.path.join(OBJ_DIR, "bench_aids.hip.o")
    cmds.append([HIPCC] + FLAGS + ["-c", BENCH_SOURCE, "-o", bench_obj])
    dec = next(s for s in SOURCES if os.path.basename(s) == "fa_decode.hip")
    want_probes = bool(probes)
    probes = {f: os.path.join(OBJ_DIR, f"fa_decode.hip.probe{f}.o") for f in (PROBE_FLAGS if want_probes else ())}
    cmds += [[HIPCC] + FLAGS + [f"-DORIN_FA_DECODE_PROBE={f}", "-c", dec, "-o", o] for f, o in probes.items()]
    pre = next(s for s in SOURCES if os.path.basename(s) == "fa_prefill.hip")
    pprobes = {f: os.path.join(OBJ_DIR, f"fa_prefill.hip.probe{f}.o") for f in (PPROBE_FLAGS if want_probes else ())}
    cmds += [[HIPCC] + FLAGS + [f"-DORIN_FA_PREFILL_PROBE={f}", "-c", pre, "-o", o] for f, o in pprobes.items()]
    with ThreadPoolExecutor(max_workers=8) as pool:
        lines = list(pool.map(_run, cmds))
    lines.append(_run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB]))
    lines.append(_run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + [stamped.get(s, o) for s, o in zip(SOURCES, objs)]
                      + ["-o", STAMPS_LIB]))
    lines.append(_run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", bench_obj, "-o", BENCH_LIB]))
    for f, o in probes.items():
        lines.append(_run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + [o if s == dec else x for s, x in zip(SOURCES, objs)]
                          + ["-o", PROBE_LIB.format(f)]))
    for f, o in pprobes.items():
        lines.append(_run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC"] + [o if s == pre else x for s, x in zip(SOURCES, objs)]
                          + ["-o", PPROBE_LIB.format(f)]))
    if verbose:
        print("\n".join(lines))
    return LIB


def probes_built():
    return all(os.path.exists(PROBE_LIB.format(f)) for f in PROBE_FLAGS) and all(os.path.exists(PPROBE_LIB.format(f)) for f in PPROBE_FLAGS)


if __name__ == "__main__":
    import sys

    print(build(verbose=True, probes="--probes" in sys.argv[1:]))
