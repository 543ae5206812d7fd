"""Build recipe: libsq_w4a16.so (HIP kernels + C ABI), the `quant` torch extension and the
benchmark's diagnostic library libsq_probes.so.

All are built in-tree, next to the `sqamd` package (the directory that is put on
sys.path so that `import quant` finds the extension):

    sparse-quant_amd/libsq_w4a16.so
    sparse-quant_amd/quant.cpython-<abi>.so
    sparse-quant_amd/libsq_probes.so

hipcc cross-compiles for gfx950 without a GPU.  Run as `python -m sqamd.build`
from sparse-quant_amd/, or call build_all().
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))  # sparse-quant_amd/
REPO_ROOT = os.path.dirname(PKG_ROOT)
CSRC = os.path.join(PKG_ROOT, "csrc")
OBJ_DIR = os.path.join(PKG_ROOT, "build")
LIB_PATH = os.path.join(PKG_ROOT, "libsq_w4a16.so")
EXT_PATH = os.path.join(PKG_ROOT, "quant" + sysconfig.get_config_var("EXT_SUFFIX"))
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

PROBES_PATH = os.path.join(PKG_ROOT, "libsq_probes.so")

HIP_SOURCES = ["sq_api.hip", "sq_dequant.hip", "sq_repack.hip", "sq_gemv2.hip", "sq_gemv_seq.hip", "sq_skinny.hip", "sq_skinny2.hip",
               "sq_skinny3.hip", "sq_gemm.hip", "sq_gemm2.hip", "sq_attn.hip", "sq_decode_attn.hip", "sq_layernorm.hip",
               "sq_lm_head.hip"]
PROBE_SOURCES = ["sq_probes.hip"]  # diagnostic kernels, a library of their own (include/sq_probes.h)
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
             # keep the compiler from forming packed-fp32 instructions
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             # the first 16 dwords of the kernel arguments arrive in scalar registers with the wave (no load
             # from the argument buffer before the first address can be formed): measured 0.19 us per launch
             # on the single-token decode kernels
             "-mllvm", "-amdgpu-kernarg-preload-count=16"]


# Kernels whose accumulators are also touched by vector arithmetic (per-group fixups, softmax
# rescaling): keep matrix-instruction results in ordinary VGPRs so that the compiler does not
# shuttle them through the accumulation registers (hundreds of v_accvgpr moves otherwise).
PER_FILE_FLAGS = {
    "sq_gemv2.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "sq_gemv_seq.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "sq_skinny2.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "sq_skinny3.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "sq_attn.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)


def build_lib(verbose=True):
    """Compile every HIP source for gfx950 and link libsq_w4a16.so and libsq_probes.so."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    sources = HIP_SOURCES + PROBE_SOURCES
    objs = [os.path.join(OBJ_DIR, s.replace(".hip", ".o")) for s in sources]

    def compile_one(pair):
        src, obj = pair
        _run([hipcc] + HIP_FLAGS + PER_FILE_FLAGS.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj])
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        list(pool.map(compile_one, zip(sources, objs)))
    n = len(HIP_SOURCES)
    for path, part in ((LIB_PATH, objs[:n]), (PROBES_PATH, objs[n:])):
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", path] + part +
             ["-Wl,-rpath," + os.path.join(ROCM, "lib")])
        if verbose:
            print("built", path)
    return LIB_PATH


def build_ext(verbose=True):
    """Compile the `quant` torch extension (host C++ only) against libsq_w4a16.so."""
    import torch
    from torch.utils import cpp_extension as ce

    inc = ce.include_paths() + [sysconfig.get_paths()["include"], os.path.join(ROCM, "include"),
                                os.path.join(REPO_ROOT, "include")]
    try:
        import pybind11
        inc.append(pybind11.get_include())
    except ImportError:
        pass
    libdirs = ce.library_paths()
    cmd = ["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=quant",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           os.path.join(CSRC, "quant_ext.cpp"), "-o", EXT_PATH]
    cmd += ["-I" + p for p in inc]
    cmd += ["-L" + p for p in libdirs] + ["-L" + PKG_ROOT]
    cmd += ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64"]
    cmd += ["-lsq_w4a16", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python"]
    cmd += ["-Wl,-rpath,$ORIGIN"] + ["-Wl,-rpath," + p for p in libdirs]
    _run(cmd)
    if verbose:
        print("built", EXT_PATH)
    return EXT_PATH


def build_all():
    build_lib()
    build_ext()


if __name__ == "__main__":
    what = sys.argv[1] if len(sys.argv) > 1 else "all"
    if what == "lib":
        build_lib()
    elif what == "ext":
        build_ext()
    else:
        build_all()
