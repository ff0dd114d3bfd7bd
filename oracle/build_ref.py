"""Build the one piece of the reference that compiles from its own source on this image
(test infrastructure): ``actnn/actnn/cpp_extension/calc_precision.cc`` - plain CPU C++
against the torch headers that ship with the installed PyTorch.  The source is compiled
where it lies under /root/reference; only the resulting module is written, into
``oracle/_ref/`` (git-ignored).  The CUDA sources of the reference need nvcc, cuRAND and
THC headers and are not buildable here.

    python oracle/build_ref.py
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
REF_SRC = "/root/reference/actnn/actnn/cpp_extension/calc_precision.cc"
OUT_DIR = os.path.join(HERE, "_ref")
MOD_NAME = "ref_calc_precision"


def build(verbose=False):
    """Returns the path of the built module, or None when the reference is not mounted."""
    if not os.path.exists(REF_SRC):
        return None
    import torch
    from torch.utils import cpp_extension as ce
    os.makedirs(OUT_DIR, exist_ok=True)
    out = os.path.join(OUT_DIR, MOD_NAME + sysconfig.get_config_var("EXT_SUFFIX"))
    if os.path.exists(out) and os.path.getmtime(out) >= os.path.getmtime(REF_SRC):
        return out                      # up to date (the torch headers take a minute to compile)
    inc = [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}"]
    libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-shared", "-fPIC", f"-DTORCH_EXTENSION_NAME={MOD_NAME}",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *inc, REF_SRC, "-o", out, f"-L{libdir}", f"-Wl,-rpath,{libdir}",
           "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10"]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return out


def load():
    """Import the prebuilt module from oracle/_ref (None if absent)."""
    import importlib.util
    import torch  # noqa: F401  (libtorch must be loaded first)
    path = os.path.join(OUT_DIR, MOD_NAME + sysconfig.get_config_var("EXT_SUFFIX"))
    if not os.path.exists(path):
        return None
    spec = importlib.util.spec_from_file_location(MOD_NAME, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


if __name__ == "__main__":
    p = build(verbose=True)
    print("built:", p)
    sys.exit(0 if p else 1)
