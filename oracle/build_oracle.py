"""Build recipe for the CPU oracle (test infrastructure, never on the product path).

Two artefacts:

* ``oracle/libsc_oracle.so``  - the plain-C restatement in ``sc_oracle.c`` (gcc).
* ``oracle/_ref/sc_extension_ref_<isa>.so`` - the reference's own CPU kernel,
  ``torch_c/sc-extension/sc.cpp``, compiled unmodified *from where it lies* under
  ``/root/reference`` with g++ against the installed torch headers.  Nothing is
  copied into the repository; the outputs are git-ignored.  Built only where the
  reference tree is present; elsewhere the prebuilt files are used as they are.

Three ISA variants of the reference are built because its bit-matmul has three
code paths selected by the preprocessor (sc.cpp:29, :132, :234): AVX-512, AVX2 and
scalar.  At run time the widest one the host CPU supports is loaded.

Run as ``python oracle/build_oracle.py [oracle|ref|all]``.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
REF_DIR = os.path.join(HERE, "_ref")
REF_SRC = "/root/reference/torch_c/sc-extension/sc.cpp"
ORACLE_LIB = os.path.join(HERE, "libsc_oracle.so")

REF_VARIANTS = {
    # name -> ISA flags handed to g++ (the reference's setup.py uses -march=native -fopenmp)
    "avx512": ["-mavx512f", "-mavx2", "-mfma"],
    "avx2": ["-mavx2", "-mfma", "-mno-avx512f"],
    "scalar": ["-mno-avx2", "-mno-avx512f"],
}


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build_oracle() -> str:
    """gcc -> oracle/libsc_oracle.so"""
    cmd = ["gcc", "-O3", "-fopenmp", "-fPIC", "-shared", "-std=c11", "-Wall", "-Wextra",
           os.path.join(HERE, "sc_oracle.c"), "-o", ORACLE_LIB, "-lm"]
    _run(cmd)
    return ORACLE_LIB


def ref_available() -> bool:
    return os.path.isfile(REF_SRC)


def ref_path(variant: str) -> str:
    return os.path.join(REF_DIR, f"sc_extension_ref_{variant}.so")


def build_ref(variants=None) -> list:
    """g++ on the reference's sc.cpp -> oracle/_ref/sc_extension_ref_<isa>.so"""
    if not ref_available():
        print("reference tree not present; keeping prebuilt oracle/_ref as is", flush=True)
        return []
    import torch
    from torch.utils import cpp_extension

    os.makedirs(REF_DIR, exist_ok=True)
    inc = [f"-I{p}" for p in cpp_extension.include_paths()]
    inc.append(f"-I{sysconfig.get_paths()['include']}")
    libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
    out = []
    for name in (variants or REF_VARIANTS):
        target = ref_path(name)
        cmd = ["g++", "-O3", "-fopenmp", "-fPIC", "-shared", "-std=c++17", "-w",
               f"-DTORCH_EXTENSION_NAME=sc_extension_ref_{name}",
               "-DTORCH_API_INCLUDE_EXTENSION_H",
               f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
               *REF_VARIANTS[name], *inc, REF_SRC, "-o", target,
               f"-L{libdir}", "-lc10", "-ltorch", "-ltorch_cpu", "-ltorch_python",
               f"-Wl,-rpath,{libdir}"]
        _run(cmd)
        out.append(target)
    return out


def main(argv):
    what = argv[1] if len(argv) > 1 else "all"
    if what in ("oracle", "all"):
        build_oracle()
    if what in ("ref", "all"):
        build_ref()


if __name__ == "__main__":
    main(sys.argv)
