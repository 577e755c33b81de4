"""In-tree build of the HIP library (libf3s_amd.so) and of the torch extension `F3S`.

    python -m fused3s_amd.build            # build both
    python -m fused3s_amd.build --lib      # only libf3s_amd.so
    python -m fused3s_amd.build --probe gather_only    # a probe library, see PROBES

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


# Probe builds: the same sources with one part of the attention step compiled out, to time what
# is left (their results are wrong on purpose). A probe library goes to
# fused3s_amd/probes/libf3s_amd_<name>.so and is used by pointing F3S_AMD_LIB at it, e.g.
#     F3S_AMD_LIB=fused3s_amd/probes/libf3s_amd_gather_only.so python bench.py --no-cpu-baseline
PROBES = {
    # K/V rows and metadata are gathered into LDS, nothing reads them back, no arithmetic
    "gather_only": ["-DF3S_PROBE_NO_COMPUTE", "-DF3S_PROBE_NO_READ"],
    # the same with every gathered row taken from the first 16384 rows (2 MiB of K, 2 MiB of V:
    # always an L2 hit) or the first 128 rows (always an L1 hit)
    "gather_only_l2_rows": ["-DF3S_PROBE_NO_COMPUTE", "-DF3S_PROBE_NO_READ",
                            "-DF3S_PROBE_ROWMASK=16383"],
    "gather_only_l1_rows": ["-DF3S_PROBE_NO_COMPUTE", "-DF3S_PROBE_NO_READ",
                            "-DF3S_PROBE_ROWMASK=127"],
    # gather and LDS reads, no arithmetic
    "no_compute": ["-DF3S_PROBE_NO_COMPUTE"],
    # LDS reads and arithmetic on whatever the first two steps left in the ring, no gather
    "no_gather": ["-DF3S_PROBE_NO_GATHER"],
}


def build_probe(name):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = [os.path.join(CSRC, s) for s in HIP_SOURCES]
    out_dir = os.path.join(HERE, "probes")
    os.makedirs(out_dir, exist_ok=True)
    out = os.path.join(out_dir, "libf3s_amd_%s.so" % name)
    _run([hipcc] + HIP_FLAGS + PROBES[name] + ["-o", out] + srcs)
    return out


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
    if "--probe" in argv:
        names = argv[argv.index("--probe") + 1:] or sorted(PROBES)
        for name in names:
            print("built", build_probe(name))
        return
    build_library()
    print("built", LIB_PATH)
    if "--lib" not in argv and os.path.exists(os.path.join(CSRC, "f3s_torch.cpp")):
        build_extension()
        print("built", EXT_PATH)


if __name__ == "__main__":
    main(sys.argv[1:])
