"""Build recipes for the native libraries (hipcc for the engine, g++ for the
synthetic-data generator).  Everything is built in-tree under deploy3d_amd/libs/.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBS = os.path.join(HERE, "libs")
ENGINE_LIB = os.path.join(LIBS, "libdeploy3d_amd.so")
SYNTH_LIB = os.path.join(LIBS, "libd3d_synth.so")

ENGINE_SOURCES = ["rulebook.hip", "conv.hip", "densify.hip", "voxelize.hip", "plugin.cpp"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
    # packed-fp32 code generation is switched off for every device function
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_engine(verbose=False):
    os.makedirs(LIBS, exist_ok=True)
    cmd = [_hipcc()] + HIPCC_FLAGS + ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    cmd += [os.path.join(CSRC, s) for s in ENGINE_SOURCES] + ["-o", ENGINE_LIB]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return ENGINE_LIB


def build_synth():
    os.makedirs(LIBS, exist_ok=True)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
           os.path.join(CSRC, "synth.cpp"), "-o", SYNTH_LIB]
    subprocess.check_call(cmd)
    return SYNTH_LIB


def build_all(verbose=False):
    build_synth()
    build_engine(verbose=verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    print("built", ENGINE_LIB, SYNTH_LIB)
