"""Build of the `fused_mlp_module` extension for MI355X (gfx950).

Counterpart of the reference's setup.py:12-45 (CUDAExtension + nvcc sm_80), in two steps:

  1. the HIP kernels and the C-ABI dispatcher (csrc/*.hip) are compiled by hipcc for gfx950 into
     `libfsw_hip.so`, which exports only the C symbols declared in include/fsw.h (and the benchmark's two
     measurement kernels, csrc/probes.hip, into `libfsw_probe.so`, include/fsw_probe.h);
  2. csrc/torch_bindings.cpp is built as a host-only C++ extension (`CppExtension`, so torch's source
     translation pass for CUDA extensions never runs) that links `libfsw_hip.so`.

Usage (in this directory):  python setup.py build_ext --inplace
`python setup.py build_hip` runs step 1 alone (the C-ABI library needs no torch).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OBJ_DIR = os.path.join(HERE, "build", "hip_obj")
LIB_NAME = "libfsw_hip.so"
HIP_SOURCES = ["kernels_pair16.hip", "kernels_tiled.hip", "kernels_skinny.hip", "kernels_stream.hip", "kernels_decode.hip", "fsw_api.hip"]
PROBE_LIB_NAME = "libfsw_probe.so"  # measurement kernels of the benchmark (include/fsw_probe.h): not part of the product
PROBE_SOURCES = ["probes.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # keep hipcc from forming packed-fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + INCLUDE, "-I" + CSRC,
]


def build_hip(verbose=True):
    """Compile csrc/*.hip for gfx950 and link libfsw_hip.so next to this file. Always recompiles."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = [s for s in HIP_SOURCES + PROBE_SOURCES if os.path.exists(os.path.join(CSRC, s))]

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        cmd = [HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        out = "\n".join(l for l in r.stdout.splitlines() if "not a recognized feature" not in l)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
        if out.strip() and verbose:
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objs = list(pool.map(compile_one, sources))
    lib = os.path.join(HERE, LIB_NAME)
    probe_objs = [o for o in objs if os.path.basename(o).replace(".o", ".hip") in PROBE_SOURCES]
    for out, members in ((lib, [o for o in objs if o not in probe_objs]), (os.path.join(HERE, PROBE_LIB_NAME), probe_objs)):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + members
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
    return lib


def main():
    if len(sys.argv) > 1 and sys.argv[1] == "build_hip":
        print(build_hip())
        return

    from setuptools import setup
    from torch.utils.cpp_extension import BuildExtension, CppExtension, include_paths

    build_hip()
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    setup(
        name="fused_mlp_module",
        ext_modules=[
            CppExtension(
                name="fused_mlp_module",
                sources=[os.path.join("csrc", "torch_bindings.cpp")],
                include_dirs=include_paths("cuda") + [INCLUDE, os.path.join(rocm, "include")],
                define_macros=[("__HIP_PLATFORM_AMD__", "1"), ("USE_ROCM", "1")],
                extra_compile_args=["-O3", "-Wall", "-std=c++17", "-Wno-unused-function"],
                library_dirs=[HERE, os.path.join(rocm, "lib")],
                libraries=["fsw_hip", "amdhip64", "c10_hip", "torch_hip"],
                extra_link_args=["-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(rocm, "lib")],
            )
        ],
        cmdclass={"build_ext": BuildExtension.with_options(use_ninja=False)},
    )


if __name__ == "__main__":
    os.chdir(HERE)
    main()
