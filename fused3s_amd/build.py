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

HIP_SOURCES = ["f3s_capi.hip", "f3s_attention.hip", "f3s_attention_wide.hip",
               "f3s_attention_units.hip", "f3s_preprocess.hip"]
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall",
    # packed-fp32 code generation is switched off for every device translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# Probe builds: the same sources with one part of the attention step compiled out, to time what
# is left (their results are wrong on purpose). A probe library goes to
# fused3s_amd/probes/libf3s_amd_<name>.so and is used by pointing F3S_AMD_LIB at it, e.g.
#     F3S_AMD_LIB=fused3s_amd/probes/libf3s_amd_gather_only.so python bench.py --no-cpu-baseline
PROBES = {
    # the column-sliced schedule's partial results through the caches instead of past them
    "partial_cached_load": ["-DF3S_PROBE_PARTIAL_CACHED_LOAD"],
    "partial_cached": ["-DF3S_PROBE_PARTIAL_CACHED_LOAD", "-DF3S_PROBE_PARTIAL_CACHED_STORE"],
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
    # column-sliced schedule: the four waves of a workgroup all compute the workgroup's first
    # unit, at the same time (what the L1 makes of rows that several waves ask for together)
    "same_unit": ["-DF3S_PROBE_SAME_UNIT"],
    # Preprocessing (window_rank_fill_kernel) with one part left out. Their block arrays are
    # incomplete: time them with `python bench.py --preprocess-only` and never hand what they
    # produce to an attention call (bench.py refuses to).
    # the compacted column ids are not enumerated from the bitset
    "pre_no_ids": ["-DF3S_PROBE_PRE_NO_IDS"],
    # no second pass over the window's edges: no ranks, rows, bitmap bits (and so no tile ids)
    "pre_no_fill": ["-DF3S_PROBE_PRE_NO_FILL"],
    # the second pass without its edgeToColumn / edgeToRow stores
    "pre_no_edge_stores": ["-DF3S_PROBE_PRE_NO_EDGE_STORES"],
    # the tile ids are not walked out of the bitmaps
    "pre_no_tile_ids": ["-DF3S_PROBE_PRE_NO_TILEIDS"],
}


def _compile_and_link(out, extra_flags, tag):
    """Every translation unit in its own hipcc process (they are independent and take most of the
    time), then one link. Objects go to build/<tag>/ and are rebuilt every time."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    obj_dir = os.path.join(HERE, "build", tag)
    os.makedirs(obj_dir, exist_ok=True)
    jobs = []
    for src in HIP_SOURCES:
        obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc] + HIP_FLAGS + extra_flags + ["-c", os.path.join(CSRC, src), "-o", obj]
        jobs.append((cmd, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE,
                                                stderr=subprocess.STDOUT, text=True)))
    objs = []
    for cmd, obj, proc in jobs:
        _report(cmd, proc.communicate()[0], proc.returncode)
        objs.append(obj)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs)
    return out


def build_probe(name):
    out_dir = os.path.join(HERE, "probes")
    os.makedirs(out_dir, exist_ok=True)
    out = os.path.join(out_dir, "libf3s_amd_%s.so" % name)
    return _compile_and_link(out, PROBES[name], "probe_" + name)


def _report(cmd, text, returncode):
    out = "\n".join(l for l in text.splitlines()
                    if "not a recognized feature for this target" not in l)
    if returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    _report(cmd, proc.stdout, proc.returncode)


def build_library():
    return _compile_and_link(LIB_PATH, [], "lib")


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
