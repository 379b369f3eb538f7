"""Builds oracle/_ref/polar_gather_ref.so: the reference's own CPU gather, compiled from the source file where it lies.

Test infrastructure only.  The reference's single host C++ file, `cache_hub/gather/gather_cpu.cpp` (a pybind11 torch
extension: `gather_kv_out_cpu(src[B,H,N,D], index[B,H,K], out[B,H,K,D])`), is compiled with g++ against the torch
headers of this image - the same thing its loader `cache_hub/gather/cpp_gather.py:10-41` does through
`torch.utils.cpp_extension.load`, written out as one compiler command.  Nothing is copied: the source is read from
`/root/reference`, the output goes to `oracle/_ref/` (git-ignored).  The rest of the reference's path is CUDA and has
no build here.

    python oracle/build_ref.py [reference_root]
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_ref")
NAME = "polar_gather_ref"


def so_path() -> str:
    return os.path.join(OUT_DIR, NAME + ".so")


def build(reference_root: str = "/root/reference", verbose: bool = False) -> str:
    """Compile and return the path of the module; raises if the reference or the compiler is missing."""
    src = os.path.join(reference_root, "cache_hub", "gather", "gather_cpu.cpp")
    if not os.path.isfile(src):
        raise FileNotFoundError(src)
    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(OUT_DIR, exist_ok=True)
    lib_dir = os.path.join(os.path.dirname(torch.__file__), "lib")
    # -O3 -std=c++17 and nothing else: the flags of the reference's loader (NDEBUG stays undefined, as there)
    cmd = ["g++", "-O3", "-std=c++17", "-shared", "-fPIC", f"-DTORCH_EXTENSION_NAME={NAME}",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    cmd += [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}"]
    cmd += [src, "-o", so_path(), f"-L{lib_dir}", f"-Wl,-rpath,{lib_dir}", "-lc10", "-ltorch_cpu", "-ltorch", "-ltorch_python"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return so_path()


def load():
    """The built module, or None when oracle/_ref has not been built."""
    if not os.path.isfile(so_path()):
        return None
    import importlib.util

    import torch  # noqa: F401  (the module links against it)

    spec = importlib.util.spec_from_file_location(NAME, so_path())
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


if __name__ == "__main__":
    print(build(*(sys.argv[1:2]), verbose=True))
