"""Builds libzoph_rnn_hip.so (the C-ABI library with the gfx950 kernels) in-tree with hipcc."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libzoph_rnn_hip.so")
SOURCES = ["zr_runtime.hip", "zr_elementwise.hip", "zr_gemm.hip", "zr_lstm.hip", "zr_softmax.hip",
           "zr_attention.hip", "zr_attn_step.hip", "zr_beam.hip", "zr_backward.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
         # packed fp32 VALU forms are kept out of the generated code on this hardware pool
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src):
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build_hip(verbose=False, jobs=4):
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, srcs))
    for _, out in results:
        if verbose and out.strip():
            print(out)
    objs = [o for o, _ in results]
    cmd = [HIPCC, "-shared", "--offload-arch=gfx950", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    return LIB




def _build_host_program(name):
    src = os.path.join(HERE, "host", name + ".cpp")
    out = os.path.join(HERE, "host", name)
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O1", "-Wall", "-o", out, src, "-L", HERE, "-lzoph_rnn_hip",
           "-Wl,-rpath,$ORIGIN/.."]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(name + " build failed:\n" + r.stdout + r.stderr)
    return out


def build_force_decode():
    """The force-decode / perplexity driver over text files (zoph_rnn_amd/host/force_decode), plain g++ against the
    C-ABI."""
    return _build_host_program("force_decode")


def build_beam_decode():
    """The beam-search translation driver over text files (zoph_rnn_amd/host/beam_decode)."""
    return _build_host_program("beam_decode")


def build_host_driver():
    """C++ test drivers of the host-side classes (tests/host/layers_forward, tests/host/train_step), plain g++
    against the C-ABI."""
    root = os.path.dirname(HERE)
    out = None
    for name in ("train_step", "layers_forward"):
        src = os.path.join(root, "tests", "host", name + ".cpp")
        out = os.path.join(root, "tests", "host", name)
        cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O1", "-Wall", "-o", out, src, "-L", HERE,
               "-lzoph_rnn_hip", "-Wl,-rpath,$ORIGIN/../../zoph_rnn_amd"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("host driver build failed:\n" + r.stdout + r.stderr)
    return out


if __name__ == "__main__":
    print(build_hip(verbose=True, jobs=int(os.environ.get("JOBS", "4"))))
