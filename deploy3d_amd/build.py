"""Build recipes for the native libraries (hipcc for the engine, g++ for the
synthetic-data generator).  Everything is built in-tree under deploy3d_amd/libs/.

Each engine source is compiled to its own object (in parallel) and the objects
are linked into one shared library.  ``build_all()`` recompiles everything;
``python -m deploy3d_amd.build --incremental`` recompiles only sources whose
text, headers or flags changed since their object was written.
"""
import concurrent.futures
import hashlib
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBS = os.path.join(HERE, "libs")
OBJ = os.path.join(LIBS, "obj")
ENGINE_LIB = os.path.join(LIBS, "libdeploy3d_amd.so")
SYNTH_LIB = os.path.join(LIBS, "libd3d_synth.so")

ENGINE_SOURCES = ["rulebook.hip", "conv.hip", "conv_half.hip", "conv_bf16.hip", "conv_int8.hip", "conv_pipe_half.hip",
                  "conv_pipe_bf16.hip", "conv_pipe_int8.hip", "densify.hip", "voxelize.hip", "scratch.hip", "plugin.cpp", "schedule.cpp"]
ENGINE_HEADERS = ["common.h", "conv_kernels.h", "conv_pipe.h", os.path.join(ROOT, "include", "d3d_spconv.h")]
# per-source extra flags
EXTRA_FLAGS = {
    # keeps the MFMA accumulators of the pipelined kernel in VGPRs (see the header of the two files)
    "conv_pipe_half.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "conv_pipe_bf16.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "conv_pipe_int8.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}
PEAKS_BIN = os.path.join(LIBS, "d3d_peaks")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # packed-fp32 code generation is switched off for every device function
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
NOISE = "is not a recognized feature for this target"


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if NOISE not in l)
    if res.returncode != 0:
        raise RuntimeError("%s failed:\n%s" % (" ".join(cmd[:1] + cmd[-3:]), out))
    return out


def _stamp(src, flags):
    h = hashlib.sha256(" ".join(flags).encode())
    for path in [os.path.join(CSRC, src)] + [p if os.path.isabs(p) else os.path.join(CSRC, p) for p in ENGINE_HEADERS]:
        if os.path.exists(path):
            with open(path, "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def _existing_sources():
    return [s for s in ENGINE_SOURCES if os.path.exists(os.path.join(CSRC, s))]


def build_engine(verbose=False, incremental=False, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    flags = HIPCC_FLAGS + ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    todo, objs = [], []
    for src in _existing_sources():
        obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        stamp = _stamp(src, flags + EXTRA_FLAGS.get(src, []))
        stamp_file = obj + ".stamp"
        fresh = False
        if incremental and os.path.exists(obj) and os.path.exists(stamp_file):
            with open(stamp_file) as f:
                fresh = f.read() == stamp
        if not fresh:
            todo.append((src, obj, stamp))

    def compile_one(item):
        src, obj, stamp = item
        out = _run([_hipcc()] + flags + EXTRA_FLAGS.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj])
        with open(obj + ".stamp", "w") as f:
            f.write(stamp)
        return src, out

    jobs = jobs or min(8, os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for src, out in pool.map(compile_one, todo):
            if verbose and out.strip():
                print(out)
    out = _run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", ENGINE_LIB])
    if verbose and out.strip():
        print(out)
    return ENGINE_LIB


def build_peaks():
    """The measured-peaks microbenchmark (dense MFMA loop, streaming copy), a standalone program bench.py runs."""
    os.makedirs(LIBS, exist_ok=True)
    _run([_hipcc(), "--offload-arch=gfx950", "-O3", "-std=c++17", os.path.join(CSRC, "peaks.hip"), "-o", PEAKS_BIN])
    return PEAKS_BIN


def build_synth():
    os.makedirs(LIBS, exist_ok=True)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
           os.path.join(CSRC, "synth.cpp"), "-o", SYNTH_LIB]
    subprocess.check_call(cmd)
    return SYNTH_LIB


def build_all(verbose=False, incremental=False):
    build_synth()
    build_engine(verbose=verbose, incremental=incremental)
    if not (incremental and os.path.exists(PEAKS_BIN) and
            os.path.getmtime(PEAKS_BIN) >= os.path.getmtime(os.path.join(CSRC, "peaks.hip"))):
        build_peaks()


if __name__ == "__main__":
    build_all(verbose=True, incremental="--incremental" in sys.argv)
    print("built", ENGINE_LIB, SYNTH_LIB)
