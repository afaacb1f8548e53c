"""Build the gfx950 selective_nd_scan libraries in-tree.

    python build.py            # C-ABI library (hipcc) + PyTorch extension (g++)
    python build.py --no-torch # C-ABI library only

Outputs (git-ignored, next to this file):
    libsnd_scan.so                      C-ABI library declared in include/snd_scan.h
    selective_nd_scan_hip_oflex*.so     thin PyTorch extension exporting fwd / bwd
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INC = os.path.join(ROOT, "include")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libsnd_scan.so")

HIP_SOURCES = ["snd_bwd_f32.hip", "snd_bwd_bf16.hip", "snd_bwd_f16.hip", "snd_wave_bwd_f32.hip", "snd_wave_bwd_bf16.hip", "snd_wave_bwd_f16.hip", "snd_wave_fwd_f32.hip", "snd_wave_fwd_bf16.hip", "snd_wave_fwd_f16.hip", "snd_fwd_f32.hip", "snd_fwd_bf16.hip",
               "snd_fwd_f16.hip", "snd_capi.hip"]
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
    # packed-FP32 VALU forms are switched off for every device function
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", INC, "-I", CSRC,
]


def run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout + "\n")
        raise RuntimeError("build step failed: " + cmd[0])
    return r.stdout


def build_capi(extra=()):
    os.makedirs(OBJ, exist_ok=True)
    extra = list(extra) + os.environ.get("SND_EXTRA_FLAGS", "").split()
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

    def one(src):
        obj = os.path.join(OBJ, src.replace(".hip", ".o"))
        out = run([hipcc, *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj])
        return obj, out

    with ThreadPoolExecutor(max_workers=8) as ex:
        res = list(ex.map(one, HIP_SOURCES))
    for _, out in res:
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip()]
        if lines:
            print("\n".join(lines))
    run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *[o for o, _ in res], "-o", LIB])
    return LIB


def build_torch_ext():
    src = os.path.join(CSRC, "snd_torch_ext.cpp")
    if not os.path.exists(src):
        return None
    import sysconfig
    import torch
    from torch.utils import cpp_extension as ce
    suffix = sysconfig.get_config_var("EXT_SUFFIX")
    out = os.path.join(HERE, "selective_nd_scan_hip_oflex" + suffix)
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=selective_nd_scan_hip_oflex", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=" + str(int(torch._C._GLIBCXX_USE_CXX11_ABI)),
           "-I", INC, "-I", "/opt/rocm/include", "-I", sysconfig.get_paths()["include"]]
    for inc in ce.include_paths():
        cmd += ["-isystem", inc]
    cmd += [src, "-o", out, "-L", HERE, "-lsnd_scan", "-Wl,-rpath,$ORIGIN",
            "-L", tlib, "-Wl,-rpath," + tlib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
            "-L", "/opt/rocm/lib", "-lamdhip64"]
    run(cmd)
    return out


def main(argv):
    extra = ["-Rpass-analysis=kernel-resource-usage"] if "--usage" in argv else []
    print("built", build_capi(extra))
    if "--no-torch" not in argv:
        ext = build_torch_ext()
        if ext:
            print("built", ext)


if __name__ == "__main__":
    main(sys.argv[1:])
