"""Build recipes for the native parts: plain compiler invocations, no build system.

  libcgnn_hip.so        device library (HIP kernels + C ABI), hipcc, gfx950 only
  libcgnn_prep.so       host-side graph preparation (C++), g++
  compressgnn_runtime   torch extension module with the reference's operator names, g++

Everything is built in-tree next to the sources so that the built files travel with
the source tree.  `python -m compressgnn_amd.build [hip|prep|runtime|all]`.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
LIB_DIR = os.path.join(HERE, "lib")

HIP_SOURCES = ["spmm.hip", "cluster.hip", "cluster_sort.hip", "transpose.hip", "merger.hip", "sample.hip", "abi.cpp"]
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # products and sums are rounded separately so that row sums match a sequential
    # CPU sum bit for bit; fused multiply-adds are written explicitly where wanted
    "-ffp-contract=off",
    # no packed-FP32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value",
]

HIP_LIB = os.path.join(LIB_DIR, "libcgnn_hip.so")
PREP_LIB = os.path.join(LIB_DIR, "libcgnn_prep.so")


def _run(cmd, cwd=None):
    print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if out.strip():
        print(out, flush=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s" % (proc.returncode, " ".join(cmd)))


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_hip():
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    procs = []
    obj_dir = os.path.join(HERE, "_obj")
    os.makedirs(obj_dir, exist_ok=True)
    for src in HIP_SOURCES:
        obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        if src.endswith(".hip"):
            cmd = [hipcc()] + HIP_FLAGS + ["-I", INCLUDE, "-I", CSRC, "-c", src, "-o", obj]
        else:
            cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-I", INCLUDE, "-I", CSRC, "-c", src, "-o", obj]
        print("+", " ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, cwd=CSRC, stdout=subprocess.PIPE,
                                            stderr=subprocess.STDOUT, text=True)))
    for cmd, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines()
                        if "packed-fp32-ops' is not a recognized feature" not in l)
        if out.strip():
            print(out, flush=True)
        if p.returncode != 0:
            raise RuntimeError("command failed (%d): %s" % (p.returncode, " ".join(cmd)))
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIB] + objs)
    return HIP_LIB


def build_prep():
    os.makedirs(LIB_DIR, exist_ok=True)
    _run(["g++", "-O3", "-std=c++17", "-fPIC", "-fopenmp", "-shared", "-I", INCLUDE,
          os.path.join(CSRC, "prep.cpp"), "-o", PREP_LIB])
    return PREP_LIB


def runtime_module_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(HERE, "compressgnn_runtime" + suffix)


def build_runtime():
    """The torch extension `compressgnn_runtime`: host code only (g++), linked against
    libcgnn_hip.so through the C ABI."""
    import torch
    from torch.utils import cpp_extension as ce
    out = runtime_module_path()
    inc = []
    for p in ce.include_paths() + [sysconfig.get_paths()["include"], INCLUDE, "/opt/rocm/include"]:
        inc += ["-I", p]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=compressgnn_runtime",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-Wno-deprecated-declarations", "-Wno-unused-result"] + inc + [
           os.path.join(CSRC, "torch_binding.cpp"), "-o", out,
           "-L", torch_lib, "-L", LIB_DIR, "-L", "/opt/rocm/lib",
           "-Wl,-rpath," + torch_lib, "-Wl,-rpath,$ORIGIN/lib", "-Wl,-rpath,/opt/rocm/lib",
           "-lcgnn_hip", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
           "-lamdhip64"]
    _run(cmd)
    return out


def build_all():
    build_hip()
    build_prep()
    build_runtime()


if __name__ == "__main__":
    what = sys.argv[1:] or ["all"]
    for w in what:
        {"hip": build_hip, "prep": build_prep, "runtime": build_runtime, "all": build_all}[w]()
