"""Build steps for the native parts: libshmt.so (HIP kernels + C ABI, hipcc,
gfx950), the ShmTensorLib pybind module (host-only C++ over the C ABI) and the
CPU oracle used by the tests. Everything is built in-tree.

    python -m shmtensor_amd.build            # build all
    python -m shmtensor_amd.build lib        # only libshmt.so
"""
import os
import shutil
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
INCLUDE = os.path.join(ROOT, "include")
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libshmt.so")
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "liboracle.so")

HIP_SOURCES = ["hashmap.hip", "fetch.hip", "scan.hip", "relabel.hip", "sample.hip", "misc.hip",
               "host_mem.hip", "errors.cc"]

MODULE_SOURCES = ["module.cc", "batch_driver.cc", "batch_sampler.cc", "host_tensors.cc"]

# Packed-FP32 instruction selection is switched off for every HIP translation
# unit (the kernels here do no floating-point arithmetic at all, rows are
# moved as raw bytes).
HIPCC_FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "not a recognized feature" not in l)
    if out.strip():
        print(out, flush=True)
    if res.returncode != 0:
        raise RuntimeError("build step failed: " + " ".join(cmd))


def hipcc():
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def build_lib():
    """One object per translation unit (compiled side by side), then one link."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, os.path.splitext(s)[0] + ".o") for s in HIP_SOURCES]

    def compile_one(pair):
        src, obj = pair
        _run([hipcc()] + HIPCC_FLAGS + ["-I" + INCLUDE, "-I" + CSRC, "-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=min(8, len(objs))) as pool:
        list(pool.map(compile_one, zip(HIP_SOURCES, objs)))
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB_PATH])
    return LIB_PATH


def module_path():
    return os.path.join(PKG, "ShmTensorLib" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_module():
    """ShmTensorLib: pybind11 surface over the C ABI. Host C++ only (g++);
    links libtorch for tensor allocation and the current-stream query."""
    import torch
    from torch.utils import cpp_extension
    tdir = os.path.dirname(torch.__file__)
    tlib = os.path.join(tdir, "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=ShmTensorLib",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for inc in cpp_extension.include_paths():
        cmd += ["-isystem", inc]
    cmd += ["-isystem", "/opt/rocm/include", "-I" + sysconfig.get_paths()["include"],
            "-I" + INCLUDE]
    cmd += [os.path.join(CSRC, "pybind", f) for f in MODULE_SOURCES]
    cmd += ["-o", module_path(),
            "-L" + tlib, "-L" + LIB_DIR, "-lshmt", "-ltorch", "-ltorch_cpu", "-ltorch_python",
            "-lc10", "-lc10_hip", "-ltorch_hip",
            "-Wl,-rpath,$ORIGIN/lib", "-Wl,-rpath," + tlib]
    _run(cmd)
    return module_path()


def build_oracle():
    """CPU oracle (test infrastructure only): plain C restatement of the
    reference algorithms, compiled with gcc."""
    src = os.path.join(ORACLE_DIR, "oracle.c")
    _run(["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-fopenmp", "-Wall", src, "-o", ORACLE_LIB,
          "-lm"])
    return ORACLE_LIB


NATIVE_TEST = os.path.join(ROOT, "tests", "native", "cabi_smoke.bin")


def build_native_test():
    """Stand-alone C++ program that drives the C ABI without Python or torch
    (run by tests/test_gpu_native.py on the GPU box)."""
    _run([hipcc(), "-O2", "-std=c++17", "-I" + INCLUDE, os.path.join(ROOT, "tests", "native", "cabi_smoke.cc"),
          "-o", NATIVE_TEST, "-L" + LIB_DIR, "-lshmt", "-Wl,-rpath,$ORIGIN/../../shmtensor_amd/lib"])
    return NATIVE_TEST


def build_all():
    build_lib()
    build_module()
    build_oracle()
    build_native_test()


if __name__ == "__main__":
    what = sys.argv[1:] or ["all"]
    for w in what:
        {"all": build_all, "lib": build_lib, "module": build_module, "oracle": build_oracle,
         "native": build_native_test}[w]()
