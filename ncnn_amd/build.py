"""Build recipe for the in-tree native libraries (hipcc cross-compiles gfx950 without a GPU)."""
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
LIBNCNNHIP = os.path.join(LIBDIR, "libncnnhip.so")

HIP_SOURCES = ["runtime.hip", "quantize.hip", "gemm_int8.hip", "gemm_int8_pipelined.hip", "conv_int8.hip", "conv_nhwc.hip", "conv_nhwc_pipelined.hip", "conv_nhwc_pipelined_split.hip", "conv_nhwc_pipelined_staged.hip", "conv_pointwise.hip", "conv_resident.hip", "conv_patch.hip", "nhwc_ops.hip", "attention.hip", "blockquant.hip", "peaks.hip"]

# -ffp-contract=off: the reference arithmetic is separate mul and add, never FMA.
# packed-fp32 ops are switched off for this pool's gfx950 parts.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-fvisibility=hidden",
               "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option"]


# per-file additions.  blockquant.hip: matrix-core results that go straight into vector arithmetic (the per-block descale) stay in
# VGPRs instead of AGPRs, which saves a register read per value (tiled kernel 135 -> 125 us at 1024 x 4096 x 4096).
# attention.hip: the same for the scores and the context on their way into the softmax arithmetic (attention core of 1500 tokens 183 -> 155 us).
HIPCC_FILE_FLAGS = {"blockquant.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"], "attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
                    "conv_pointwise.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"], "conv_resident.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _run(cmd):
    print("+ " + " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_kernels(jobs=8):
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(ROOT, "build", "obj")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    for src in HIP_SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = ["hipcc"] + HIPCC_FLAGS + HIPCC_FILE_FLAGS.get(src, []) + ["-I", os.path.join(ROOT, "include"), "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        print("+ " + " ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd)))
        if len(procs) >= jobs:
            s, p = procs.pop(0)
            if p.wait() != 0:
                raise RuntimeError("hipcc failed on " + s)
    for s, p in procs:
        if p.wait() != 0:
            raise RuntimeError("hipcc failed on " + s)
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIBNCNNHIP] + objs)
    return LIBNCNNHIP


HOST_SOURCES = ["ncnn/allocator.cpp", "ncnn/mat.cpp", "ncnn/option.cpp", "ncnn/datareader.cpp", "ncnn/paramdict.cpp", "ncnn/modelbin.cpp", "ncnn/hipmat.cpp",
                "ncnn/layer.cpp", "ncnn/net.cpp", "layers/glue_layers.cpp", "layers/hip_support.cpp", "layers/convolution_hip.cpp",
                "layers/innerproduct_hip.cpp", "layers/gemm_hip.cpp", "layers/multiheadattention_hip.cpp", "c_api.cpp", "c_api_layer.cpp"]
LIBNCNN_AMD = os.path.join(LIBDIR, "libncnn_amd.so")
LIBNCNN_AMD_ASAN = os.path.join(LIBDIR, "libncnn_amd_asan.so")

# strict IEEE on the host too: the load-time weight quantiser and the scale folding must round
# exactly like the reference's scalar code
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-fopenmp", "-fno-fast-math", "-ffp-contract=off", "-fvisibility=hidden", "-Wall", "-Wextra",
              "-Wno-unused-parameter"]


def build_host(sanitize=False):
    """libncnn_amd.so: the ncnn-API mirror (Mat, ParamDict, ModelBin, Net, Extractor), the four HIP layers and the C API.
    It links against libncnnhip.so, which carries the kernels.
    sanitize=True builds libncnn_amd_asan.so beside it with AddressSanitizer and UBSan on the host code (there is no GPU
    code in this library).  Run the CPU tests on it with
      LD_PRELOAD=$(gcc -print-file-name=libasan.so) ASAN_OPTIONS=detect_leaks=0 NCNN_AMD_HOST_LIB=<that file> python -m pytest tests -m "not gpu"
    """
    hostdir = os.path.join(PKG, "host")
    srcs = [os.path.join(hostdir, s) for s in HOST_SOURCES]
    out = LIBNCNN_AMD_ASAN if sanitize else LIBNCNN_AMD
    flags = HOST_FLAGS + (["-g", "-fsanitize=address,undefined", "-fno-omit-frame-pointer"] if sanitize else [])
    _run(["g++"] + flags + ["-I", os.path.join(ROOT, "include"), "-I", hostdir, "-shared", "-o", out] + srcs
         + ["-L", LIBDIR, "-lncnnhip", "-Wl,-rpath,$ORIGIN"])
    return out


LIBPLUGIN = os.path.join(LIBDIR, "libncnnhip_plugin.so")


def build_plugin(c_api_include=None):
    """libncnnhip_plugin.so from plugin/ncnnhip_plugin.c: the four int8 layers written against ncnn's public C API only.
    Without arguments it is compiled against this repository's copy of that API and linked to libncnn_amd.so (what the tests
    load); with c_api_include = the directories that hold an ncnn build's c_api.h, platform.h and ncnn_export.h it is compiled
    against those and left to resolve the ncnn_* symbols from the libncnn the host program links."""
    src = os.path.join(ROOT, "plugin", "ncnnhip_plugin.c")
    cmd = ["gcc", "-std=c99", "-O2", "-fPIC", "-shared", "-fvisibility=hidden", "-fno-fast-math", "-ffp-contract=off", "-Wall", "-Wextra",
           "-I", os.path.join(ROOT, "include")]
    if c_api_include:
        cmd += [x for d in c_api_include for x in ("-I", d)]
        cmd += [src, "-o", LIBPLUGIN, "-L", LIBDIR, "-lncnnhip", "-lm", "-lpthread", "-Wl,-rpath,$ORIGIN"]
    else:
        cmd += ["-DNCNNHIP_PLUGIN_AGAINST_NCNN_AMD", src, "-o", LIBPLUGIN, "-L", LIBDIR, "-lncnn_amd", "-lncnnhip", "-lm", "-lpthread",
                "-Wl,-rpath,$ORIGIN"]
    _run(cmd)
    return LIBPLUGIN


def build_all():
    build_kernels()
    build_host()
    build_plugin()


if __name__ == "__main__":
    if "--asan-host" in sys.argv:
        print("built", build_host(sanitize=True))
        sys.exit(0)
    build_all()
    print("built", LIBNCNNHIP)
    sys.exit(0)
