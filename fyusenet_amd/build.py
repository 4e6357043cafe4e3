"""Builds libfynhip.so (HIP kernels + host engine + C ABI) for gfx950 with hipcc, in-tree."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.environ.get("FYNHIP_BUILD_LIB", os.path.join(HERE, "libfynhip.so"))  # experimental builds go elsewhere
CONV_PARTS = 8  # conv_mfma.hip is compiled this many times, each time with a slice of the tile table
SOURCES = ["layers_direct.hip", "conv_rows.hip", "conv_h16.hip", "conv_d16.hip", "engine.cpp", "conv_plan.cpp", "fusion.cpp", "layers.cpp", "api.cpp"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
EXTRA = os.environ.get("FYNHIP_EXTRA_FLAGS", "").split()  # e.g. -D switches of experimental builds
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-result",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose=True, jobs=8):
    objdir = os.path.join(HERE, "_obj") if "FYNHIP_BUILD_LIB" not in os.environ else LIB + ".obj"
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    units = [("conv_mfma.hip", "conv_mfma.part%d.o" % i, ["-DFYN_CONV_PARTS=%d" % CONV_PARTS, "-DFYN_CONV_PART=%d" % i])
             for i in range(CONV_PARTS)]
    # conv_p16.hip once per storage type (fp32 tensors with the host entry points, fp16 tensors)
    units += [("conv_p16.hip", "conv_p16.f32.o", ["-DFYN_P16_HALF=0"]), ("conv_p16.hip", "conv_p16.f16.o", ["-DFYN_P16_HALF=1"])]
    units += [(src, src + ".o", []) for src in SOURCES]
    for src, objname, defs in units:
        obj = os.path.join(objdir, objname)
        objs.append(obj)
        cmd = [HIPCC] + FLAGS + EXTRA + defs + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((objname, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,--no-undefined", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            sys.stderr.write(out + "\n")
            raise RuntimeError("hipcc failed on %s" % src)
        if out.strip():
            print(out)


def build_cpp_example(verbose=True):
    """Compiles tests/cpp/surface_example.cpp, a program written against the C++ description surface of
    include/fynhip.hpp, and links it with libfynhip.so (host compiler only; the GPU tests run it)."""
    root = os.path.dirname(HERE)
    outdir = os.path.join(root, "tests", "cpp", "_build")
    os.makedirs(outdir, exist_ok=True)
    exe = os.path.join(outdir, "surface_example")
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O1", "-Wall", "-Wextra", "-I", os.path.join(root, "include"),
           os.path.join(root, "tests", "cpp", "surface_example.cpp"), "-o", exe, "-L", HERE, "-lfynhip",
           "-Wl,-rpath,$ORIGIN/../../../fyusenet_amd", "-Wl,--allow-shlib-undefined"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return exe


if __name__ == "__main__":
    build()
    build_cpp_example()
