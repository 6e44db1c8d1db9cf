"""In-tree build of the native parts: libdmm.so (HIP kernels + C ABI, hipcc, gfx950) and
_C.so (the PyTorch operator, host C++ only, g++).  No hipify, no JIT cache: the built files
sit next to this module so they travel with the tree.

    python -m decode_matmul_amd.build            # build both
    python -m decode_matmul_amd.build --lib      # only libdmm.so
"""
import os
import re
import shutil
import subprocess
import sys
import sysconfig

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(ROOT, "include")
LIB_PATH = os.path.join(PKG_DIR, "libdmm.so")
EXT_PATH = os.path.join(PKG_DIR, "_C.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # scalar fp32 code must not be turned into packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines()
        if "'-packed-fp32-ops' is not a recognized feature" not in line   # host pass, harmless
    )
    if proc.returncode != 0:
        raise RuntimeError("build command failed (%d):\n%s\n%s" % (proc.returncode, " ".join(cmd), out))
    return out


def hipcc_path():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def build_lib(verbose=False):
    """hipcc: csrc/dmm.hip (which includes the dmm_*.h kernel files beside it) -> libdmm.so
    (gfx950 code object + the extern "C" entry points)."""
    cmd = [hipcc_path()] + HIPCC_FLAGS + ["-Rpass-analysis=kernel-resource-usage",
                                          "-I" + INCLUDE, "-o", LIB_PATH, os.path.join(CSRC, "dmm.hip")]
    out = _run(cmd)
    # No kernel may spill registers to scratch memory: the kernels are sized to their register
    # budget, and a build of the streaming kernel that spilled ran at half speed and returned
    # wrong sums on the GPU.  The compiler's resource remarks name the offender.
    name, spilled = None, []
    for line in out.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line:
            if int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0]) != 0:
                spilled.append(name)
    if spilled:
        os.remove(LIB_PATH)
        raise RuntimeError("kernels spill registers to scratch memory: %s" % ", ".join(spilled))
    rest, held, skip = [], [], 0
    for line in out.splitlines():   # drop the remarks, the include trail ahead of each and the
        if line.startswith("In file included from "):   # two source-context lines after it
            held.append(line)
            continue
        if "-Rpass-analysis=kernel-resource-usage" in line:
            held, skip = [], 2
        elif skip and re.match(r"^\s*\d*\s*\|", line):
            skip -= 1
        else:
            skip = 0
            rest += held + [line]
            held = []
    rest = "\n".join(rest)
    if verbose and rest.strip():
        print(rest)
    return LIB_PATH


def build_ext(verbose=False):
    """g++: csrc/torch_binding.cpp -> _C.so, linked against libdmm.so (rpath $ORIGIN)."""
    import torch
    from torch.utils import cpp_extension as ce

    if not os.path.exists(LIB_PATH):
        build_lib(verbose)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    inc = ce.include_paths() + [sysconfig.get_paths()["include"], os.path.join(rocm, "include"), INCLUDE]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [
        shutil.which("g++") or "g++",
        "-O2", "-std=c++17", "-fPIC", "-shared",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C",
        "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
        "-Wno-deprecated-declarations",
    ]
    cmd += ["-isystem" + p for p in inc]
    cmd += [os.path.join(CSRC, "torch_binding.cpp"), "-o", EXT_PATH]
    cmd += ["-L" + torch_lib, "-L" + PKG_DIR, "-ldmm", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip",
            "-ltorch", "-ltorch_python", "-Wl,-rpath,$ORIGIN", "-Wl,--no-as-needed"]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return EXT_PATH


def build_all(verbose=False):
    build_lib(verbose)
    build_ext(verbose)
    return LIB_PATH, EXT_PATH


if __name__ == "__main__":
    if "--lib" in sys.argv:
        print(build_lib(True))
    else:
        print(*build_all(True), sep="\n")
