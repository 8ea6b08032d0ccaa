"""Builds the native libraries of this package in-tree for gfx950.

    python pytorch_cluster_amd/build.py [--jobs N] [--skip-torch-ops]

(run as a script: importing the package needs the libraries built here)

Outputs (next to this file, git-ignored):
  libpca_neighbors.so   HIP kernels + the C ABI of include/pca_neighbors.h
  _torch_ops.so         TorchScript operator binding (links the above)
  libpca_probe.so       csrc/probes/: measurement and checking aids
                        (`bench.py --probe`, the bf16 rounding check of
                        tests/test_gpu_dtypes.py), no part of the searches
"""
import argparse
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "_build")
CAPI_LIB = os.path.join(HERE, "libpca_neighbors.so")
TORCH_OPS_LIB = os.path.join(HERE, "_torch_ops.so")
PROBE_LIB = os.path.join(HERE, "libpca_probe.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# Packed FP32 instructions are switched off for every device compile.  Matrix
# core results are compared by the vector ALU right away, so they are kept in
# ordinary vector registers (no accumulator-register copies).
HIP_FLAGS = [
    "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument",
] + os.environ.get("PCA_EXTRA_HIP_FLAGS", "").split()


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True)
    # the host pass does not know the packed-fp32 feature; that is harmless
    out = "\n".join(line for line in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in line)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _compile_hip(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    _run([HIPCC] + HIP_FLAGS + ["-c", src, "-o", obj])
    return obj


# The host (CPU) searches: plain C++, fused multiply-adds and 8-wide vectors
# (checked for at run time).
HOST_SOURCES = ["cpu_search.cpp"]
HOST_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-mavx2", "-mfma", "-pthread",
              "-fno-math-errno", "-Wall"]


def _compile_host(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    _run(["g++"] + HOST_FLAGS + ["-c", src, "-o", obj])
    return obj


def build_capi(jobs):
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    host = [os.path.join(CSRC, name) for name in HOST_SOURCES]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        host_objects = [pool.submit(_compile_host, src) for src in host]
        objects = list(pool.map(_compile_hip, sources))
        objects += [f.result() for f in host_objects]
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-pthread",
          "-o", CAPI_LIB] + objects)
    return CAPI_LIB


def build_probes():
    sources = sorted(glob.glob(os.path.join(CSRC, "probes", "*.hip")))
    _run([HIPCC] + HIP_FLAGS + ["-shared"] + sources + ["-o", PROBE_LIB])
    return PROBE_LIB


def build_torch_ops():
    import torch
    from torch.utils import cpp_extension

    includes = []
    for path in cpp_extension.include_paths():
        includes += ["-I", path]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
        "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi, "-Wno-deprecated-declarations",
        "-I", "/opt/rocm/include",
    ] + includes + [
        os.path.join(CSRC, "torch_ops.cpp"), "-o", TORCH_OPS_LIB,
        "-L", HERE, "-lpca_neighbors",
        "-L", torch_lib, "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10",
        "-lc10_hip", "-lamdhip64",
        "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib,
    ]
    _run(cmd)
    return TORCH_OPS_LIB


def note_commit():
    """Writes the commit the libraries are built from next to them (for the
    benchmark line; the GPU box gets the tree without its history)."""
    repo = os.path.dirname(HERE)
    try:
        head = subprocess.run(["git", "-C", repo, "rev-parse", "--short",
                               "HEAD"], capture_output=True, text=True,
                              check=True).stdout.strip()
        dirty = subprocess.run(["git", "-C", repo, "status", "--porcelain",
                                "--untracked-files=no"], capture_output=True,
                               text=True, check=True).stdout.strip()
    except (OSError, subprocess.CalledProcessError):
        return
    with open(os.path.join(HERE, "build_commit.txt"), "w") as f:
        f.write(head + ("+" if dirty else "") + "\n")


def build_all(jobs=None, torch_ops=True):
    jobs = jobs or min(8, os.cpu_count() or 1)
    note_commit()
    build_capi(jobs)
    build_probes()
    if torch_ops:
        build_torch_ops()


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=None)
    ap.add_argument("--skip-torch-ops", action="store_true")
    args = ap.parse_args(argv)
    build_all(args.jobs, not args.skip_torch_ops)
    print("built", CAPI_LIB)
    if not args.skip_torch_ops:
        print("built", TORCH_OPS_LIB)


if __name__ == "__main__":
    sys.exit(main())
