"""Build recipe for oracle/_ref: the reference's own CPU extension modules.

TEST INFRASTRUCTURE ONLY.  Compiles, with g++ and nothing else, the CPU-only
translation units of the reference checkout (default /root/reference) exactly
where they lie, against the torch headers of this image, the way the
reference's package/setup.py:36-45 does for a machine without CUDA
(-D__NO_CUDA__, -fopenmp, -O3).  Outputs go to oracle/_ref/ only; no
reference source is copied.  The resulting pybind modules are used by tests to
validate the C restatement in oracle/ and by the bench as the timed CPU
baseline.  When the reference checkout is absent this script does nothing and
whatever was built earlier is used as is.
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "_ref")

# module name -> source basename (package/setup.py:64-79 of the reference)
MODULES = {
    "_mapped_convolution": "mapped_convolution_layer",
    "_mapped_transposed_convolution": "mapped_transposed_convolution_layer",
    "_mapped_max_pooling": "mapped_max_pooling_layer",
    "_mapped_avg_pooling": "mapped_avg_pooling_layer",
    "_resample": "resample_layer",
    "_weighted_mapped_convolution": "weighted_mapped_convolution_layer",
    "_weighted_mapped_transposed_convolution":
        "weighted_mapped_transposed_convolution_layer",
    "_weighted_mapped_max_pooling": "weighted_mapped_max_pooling_layer",
    "_weighted_mapped_avg_pooling": "weighted_mapped_avg_pooling_layer",
    "_weighted_resample": "weighted_resample_layer",
}


# the host-side icosphere tools (package/setup.py:86-94): one source under src/util/cpp
UTIL_MODULES = {"_sphere": "sphere"}


def _compile(ref_root, name, base, verbose, subdir="nn"):
    import torch
    from torch.utils import cpp_extension as ce
    src = os.path.join(ref_root, "package/ext_modules/src", subdir, "cpp", base + ".cpp")
    inc = os.path.join(ref_root, "package/ext_modules/include")
    out = os.path.join(OUT, name + ".so")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-std=c++17", "-O3", "-fopenmp", "-fPIC", "-shared", "-w",
           "-D__NO_CUDA__", "-DTORCH_EXTENSION_NAME=" + name,
           "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + inc, "-I" + sysconfig.get_paths()["include"]]
    cmd += ["-I" + p for p in ce.include_paths()]
    cmd += [src, "-o", out, "-L" + torch_lib, "-Wl,-rpath," + torch_lib,
            "-lc10", "-ltorch_cpu", "-ltorch", "-ltorch_python"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


def build(ref_root="/root/reference", verbose=False, jobs=4):
    """Compile every module; returns the list of .so files (empty if no reference)."""
    if not os.path.isdir(os.path.join(ref_root, "package/ext_modules/src/nn/cpp")):
        return []
    os.makedirs(OUT, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        futs = [ex.submit(_compile, ref_root, n, b, verbose) for n, b in MODULES.items()]
        futs += [ex.submit(_compile, ref_root, n, b, verbose, "util")
                 for n, b in UTIL_MODULES.items()]
        return [f.result() for f in futs]


if __name__ == "__main__":
    built = build(verbose=True)
    print("built %d reference CPU modules into %s" % (len(built), OUT))
    sys.exit(0)
