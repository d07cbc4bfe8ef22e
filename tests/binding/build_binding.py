"""Builds tests/binding/rpu_base_tiles_amd.cpp (pybind11 + libtorch, host code only) against include/rpu_amd.h and
aihwkit_amd/lib/librpu_amd.so into tests/binding/build/.  ``python tests/binding/build_binding.py`` builds ahead of a
GPU run; the tests call ``build()``, which compiles only when the module is missing or older than its sources."""
import os
import subprocess
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SOURCE = os.path.join(HERE, "rpu_base_tiles_amd.cpp")
HEADER = os.path.join(ROOT, "include", "rpu_amd.h")
LIB_DIR = os.path.join(ROOT, "aihwkit_amd", "lib")
OUT_DIR = os.path.join(HERE, "build")
MODULE = os.path.join(OUT_DIR, "rpu_base_tiles_amd" + sysconfig.get_config_var("EXT_SUFFIX"))


def command():
    import pybind11
    import torch
    from torch.utils import cpp_extension as ce
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [hipcc, "-x", "c++", "-std=c++17", "-O1", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for inc in ce.include_paths("cuda") + [pybind11.get_include(), sysconfig.get_paths()["include"],
                                           os.path.join(ROOT, "include")]:
        cmd += ["-I", inc]
    cmd += [SOURCE, "-o", MODULE, "-L", torch_lib, "-L", LIB_DIR, "-lrpu_amd", "-lc10", "-lc10_hip", "-ltorch_cpu",
            "-ltorch_hip", "-ltorch", "-ltorch_python", "-Wl,-rpath," + torch_lib, "-Wl,-rpath,$ORIGIN/../../../aihwkit_amd/lib"]
    return cmd


def build(force=False):
    """Path of the built module; compiles when it is missing or older than the source, the header or the library."""
    deps = [SOURCE, HEADER, os.path.join(LIB_DIR, "librpu_amd.so"), os.path.abspath(__file__)]
    if not force and os.path.exists(MODULE) and all(os.path.getmtime(MODULE) >= os.path.getmtime(d) for d in deps):
        return MODULE
    os.makedirs(OUT_DIR, exist_ok=True)
    done = subprocess.run(command(), capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError("building the binding failed:\n" + done.stdout[-4000:] + done.stderr[-8000:])
    return MODULE


def load():
    """The built module, imported from its file."""
    import importlib.util
    import torch  # noqa: F401  (libtorch must be loaded before the extension)
    spec = importlib.util.spec_from_file_location("rpu_base_tiles_amd", build())
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


if __name__ == "__main__":
    print(build(force=True))
