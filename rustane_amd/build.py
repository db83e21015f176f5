"""Build steps for the native parts: the gfx950 decode library and the host engine above it."""
import os
import subprocess

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "csrc")
LIBDIR = os.path.join(ROOT, "lib")
HIPDECODE_SO = os.path.join(LIBDIR, "libhipdecode.so")
ENGINE_SO = os.path.join(LIBDIR, "librustane_engine.so")
GENERATE_BIN = os.path.join(LIBDIR, "generate")
SERVE_BIN = os.path.join(LIBDIR, "serve")

HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-fopenmp", "-Wall"]


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("build step failed: %s\n%s" % (" ".join(cmd), res.stdout))
    return res.stdout


def build_hipdecode():
    os.makedirs(LIBDIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _run([hipcc] + HIP_FLAGS + [os.path.join(CSRC, "hip_decode.hip"), "-o", HIPDECODE_SO])
    return HIPDECODE_SO


def engine_sources():
    d = os.path.join(CSRC, "engine")
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(".cc") and not f.endswith("_main.cc"))


def build_engine():
    """Host engine (session API, samplers, synthetic weights); links against libhipdecode.so."""
    os.makedirs(LIBDIR, exist_ok=True)
    inc = os.path.join(os.path.dirname(ROOT), "include")
    _run(["g++"] + CXX_FLAGS + ["-shared", "-I", inc] + engine_sources() +
         ["-o", ENGINE_SO, "-L", LIBDIR, "-lhipdecode", "-Wl,-rpath,$ORIGIN"])
    for src, out in (("generate_main.cc", GENERATE_BIN), ("serve_main.cc", SERVE_BIN)):
        _run(["g++"] + CXX_FLAGS + ["-I", inc, os.path.join(CSRC, "engine", src), "-o", out, "-L", LIBDIR,
                                    "-lrustane_engine", "-lhipdecode", "-Wl,-rpath,$ORIGIN"])
    return ENGINE_SO


def build_all():
    build_hipdecode()
    build_engine()
