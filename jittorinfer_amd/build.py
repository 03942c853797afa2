"""Builds jittorinfer_amd/libggml-hip-mla.so (HIP kernels + C ABI + ggml backend plugin) for gfx950 with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libggml-hip-mla.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
          # packed-fp32 instruction forms are kept out of the device code
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-Wno-unused-command-line-argument"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose=False):
    objs = []
    for src in ("mla_kernels.hip", "mla_decode_kernel.hip", "mla_kv_write.hip", "mla_front.hip", "ggml_mla_backend.cpp", "mla_page_table.cpp"):
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        cmd = [HIPCC] + COMMON + (["-x", "hip"] if src == "ggml_mla_backend.cpp" else []) + ["-c", os.path.join(CSRC, src), "-o", obj]
        out = _run(cmd)
        if verbose and out.strip():
            print(out)
        objs.append(obj)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-ldl"])
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
