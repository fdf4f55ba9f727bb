"""Build recipe of the HIP library: hipcc, gfx950 only, in-tree output (tab_amd/lib/)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libtab_amd.so")
SOURCES = ["tab_capi.hip", "tab_conv.hip", "tab_conv_mfma_tnn.hip", "tab_conv_mfma_tbn.hip", "tab_conv_mfma_btn.hip",
           "tab_conv_mfma_bnn.hip", "tab_conv_mfma_drf.hip", "tab_conv_mfma_rtn.hip", "tab_conv_fused1x1.hip", "tab_quantize.hip"]
OBJ_DIR = os.path.join(LIB_DIR, "obj")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops: keep the compiler from forming packed-FP32 VALU ops from float code.
# -Werror=pass-failed: a kernel whose amdgpu_waves_per_eu request the compiler cannot meet fails the build, so that the
# residency the shape model counts on is the residency that was compiled.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-result", "-Werror=pass-failed",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


PEAK_SRC = os.path.join(CSRC, "valu_peak.hip")
PEAK_BIN = os.path.join(LIB_DIR, "valu_peak")


def build_valu_peak():
    """Standalone microbenchmark of the VALU issue rates the conv roofline is priced with."""
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [HIPCC] + HIP_FLAGS + ["-o", PEAK_BIN, PEAK_SRC]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout)
    return PEAK_BIN


MFMA_PEAK_SRC = os.path.join(CSRC, "mfma_peak.hip")
MFMA_PEAK_BIN = os.path.join(LIB_DIR, "mfma_peak")


def build_mfma_peak():
    """Standalone microbenchmark of the FP4 matrix-core rate with and without operand expansion."""
    os.makedirs(LIB_DIR, exist_ok=True)
    _hipcc([HIPCC] + HIP_FLAGS + ["-o", MFMA_PEAK_BIN, MFMA_PEAK_SRC])
    return MFMA_PEAK_BIN


def extension_path():
    import sysconfig

    return os.path.join(HERE, "_C" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_torch_extension(verbose=False):
    """Compile csrc/torch_binding.cpp (host code only: g++, no hipify, no HIP sources) into the
    CPython extension tab_amd/_C, linked against libtab_amd.so and the torch libraries."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    includes = cpp_extension.include_paths() + [sysconfig.get_paths()["include"], "/opt/rocm/include"]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=_C", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    cmd += ["-I" + i for i in includes]
    cmd += [os.path.join(CSRC, "torch_binding.cpp"), "-o", extension_path(), "-L" + torch_lib, "-L" + LIB_DIR,
            "-ltab_amd", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
            "-Wl,-rpath,$ORIGIN/lib", "-Wl,-rpath," + torch_lib]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("g++ failed:\n" + proc.stdout)
    if verbose and proc.stdout.strip():
        print(proc.stdout)
    return extension_path()


def _hipcc(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed: " + " ".join(cmd) + "\n" + out)
    return out


def build_library(verbose=False):
    """Compile every HIP source (one hipcc per source, side by side) and link libtab_amd.so.
    Always recompiles."""
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = [os.path.join(OBJ_DIR, s.replace(".hip", ".o")) for s in SOURCES]
    cmds = [[HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=min(8, len(cmds))) as pool:
        outs = list(pool.map(_hipcc, cmds))
    outs.append(_hipcc([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs))
    if verbose and any(o.strip() for o in outs):
        print("\n".join(o for o in outs if o.strip()))
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_valu_peak())
    print(build_mfma_peak())
    print(build_torch_extension(verbose=True))
