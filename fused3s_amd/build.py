"""In-tree build of the HIP library (libf3s_amd.so) and of the torch extension `F3S`.

    python -m fused3s_amd.build            # build both
    python -m fused3s_amd.build --lib      # only libf3s_amd.so

hipcc cross-compiles for gfx950 without a GPU; the built files stay next to the package so
that they travel with the source tree.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libf3s_amd.so")
EXT_PATH = os.path.join(HERE, "F3S" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))

HIP_SOURCES = ["f3s_capi.hip", "f3s_attention.hip", "f3s_attention_units.hip", "f3s_preprocess.hip"]
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wall",
    # packed-fp32 code generation is switched off for every device translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)


def build_library():
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = [os.path.join(CSRC, s) for s in HIP_SOURCES]
    _run([hipcc] + HIP_FLAGS + ["-o", LIB_PATH] + srcs)
    return LIB_PATH


def build_extension():
    """Compile csrc/f3s_torch.cpp (host C++ only) against torch and link it to libf3s_amd.so."""
    import torch
    from torch.utils import cpp_extension

    incs = cpp_extension.include_paths()
    incs += ["/opt/rocm/include", sysconfig.get_paths()["include"]]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1",
           "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=F3S", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for i in incs:
        cmd += ["-isystem", i]
    cmd += [os.path.join(CSRC, "f3s_torch.cpp"), "-o", EXT_PATH,
            "-L" + HERE, "-lf3s_amd", "-L" + torch_lib, "-lc10", "-lc10_hip", "-ltorch_cpu",
            "-ltorch_hip", "-ltorch", "-ltorch_python", "-L/opt/rocm/lib", "-lamdhip64",
            "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib]
    _run(cmd)
    return EXT_PATH


def main(argv):
    build_library()
    print("built", LIB_PATH)
    if "--lib" not in argv and os.path.exists(os.path.join(CSRC, "f3s_torch.cpp")):
        build_extension()
        print("built", EXT_PATH)


if __name__ == "__main__":
    main(sys.argv[1:])
