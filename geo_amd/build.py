"""In-tree build of the native code: ``python -m geo_amd.build``.

* ``geo_amd/lib/libgeo_sc.so``            - HIP kernels + C ABI (hipcc, gfx950 only)
* ``geo_amd/lib/libgeo_sc_probe.so``      - the benchmark's instruction issue-rate probe
* ``geo_amd/lib/sc_extension_cuda*.so``   - PyTorch module with the reference's GPU op names
* ``geo_amd/lib/sc_extension*.so``        - PyTorch module with the reference's CPU op name
                                           (runs the same GPU kernels)
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
INCLUDE = os.path.join(ROOT, "include")

HIP_SOURCES = ["sc_streams.hip", "sc_conv_fwd.hip", "sc_conv_bwd.hip", "sc_epilogue.hip", "sc_api.hip"]
PROBE_SOURCE = "sc_probe.hip"   # the benchmark's issue-rate probe: a library of its own, outside the C ABI
TORCH_MODULES = {"sc_extension_cuda": "sc_extension_cuda.cpp", "sc_extension": "sc_extension.cpp"}

# gfx950 only; packed-FP32 instruction selection is switched off for every device pass
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-fvisibility=hidden",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               f"-I{INCLUDE}", f"-I{CSRC}"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if out:
        print(out, flush=True)
    if res.returncode != 0:
        raise RuntimeError(f"command failed ({res.returncode}): {' '.join(cmd)}")


def lib_path() -> str:
    return os.path.join(LIBDIR, "libgeo_sc.so")


def module_path(name: str) -> str:
    return os.path.join(LIBDIR, name + sysconfig.get_config_var("EXT_SUFFIX"))


def build_hip_library() -> str:
    os.makedirs(OBJDIR, exist_ok=True)
    sources = [s for s in HIP_SOURCES if os.path.isfile(os.path.join(CSRC, s))]
    objs = [os.path.join(OBJDIR, s.replace(".hip", ".o")) for s in sources]
    with ThreadPoolExecutor(max_workers=4) as ex:
        list(ex.map(lambda so: _run(["hipcc", *HIPCC_FLAGS, "-c", os.path.join(CSRC, so[0]), "-o", so[1]]),
                    zip(sources, objs)))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", lib_path()])
    _run(["hipcc", *HIPCC_FLAGS, "-shared", os.path.join(CSRC, PROBE_SOURCE), "-o",
          os.path.join(LIBDIR, "libgeo_sc_probe.so")])
    return lib_path()


def build_torch_modules() -> list:
    import torch
    from torch.utils import cpp_extension

    inc = [f"-I{p}" for p in cpp_extension.include_paths()]
    inc += [f"-I{sysconfig.get_paths()['include']}", f"-I{INCLUDE}", f"-I{CSRC}", "-I/opt/rocm/include"]
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")

    def one(item):
        name, src = item
        out = module_path(name)
        _run(["g++", "-O2", "-fPIC", "-shared", "-std=c++17", "-w",
              "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-DTORCH_EXTENSION_NAME={name}",
              "-DTORCH_API_INCLUDE_EXTENSION_H",
              f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
              *inc, os.path.join(CSRC, src), "-o", out,
              f"-L{LIBDIR}", "-lgeo_sc", f"-L{tlib}", "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip",
              "-ltorch_python", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}"])
        return out

    with ThreadPoolExecutor(max_workers=2) as ex:
        return list(ex.map(one, TORCH_MODULES.items()))


def build_all():
    build_hip_library()
    build_torch_modules()


if __name__ == "__main__":
    build_all()
