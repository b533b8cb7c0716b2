"""In-tree build of the polyrl_amd HIP extensions for gfx950 (MI355X).

    PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace

Two modules land next to the package so they travel with a repo snapshot to
GPU boxes: ``polyrl_amd._hip`` (dense-decoder engine + trainer kernels) and
``polyrl_amd._hip_seq`` (sequence-mixer kernels of the hybrid decoders).
``POLYRL_EXT=seq`` (or ``core``) builds only that one.
"""
import glob
import os

os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")

# hipify writes *_hip.hip copies of each source; a header-only edit does not
# refresh them, which leaves stale objects in incremental builds. Remove the
# copies so every build re-derives them from the true sources.
for _f in glob.glob(os.path.join("polyrl_amd", "ops", "csrc", "*_hip.hip")):
    os.remove(_f)

from setuptools import setup
from torch.utils.cpp_extension import BuildExtension, CUDAExtension

CSRC = os.path.join("polyrl_amd", "ops", "csrc")

CORE = ("bindings.cpp", "gemm_tuned.cpp", "elementwise.hip",
        "rmsnorm_train.hip", "rope_train.hip", "logprobs.hip", "sampling.hip",
        "kv_cache.hip", "attention_decode.hip", "attention_prefill.hip",
        "attention_backward.hip", "attention_backward_v3.hip")
SEQ = ("seq_bindings.cpp", "seq_ops.hip", "seq_scan.hip", "seq_attn.hip",
       "seq_moe.hip", "seq_attn_mfma.hip", "seq_gqa.hip", "seq_gqa_mfma.hip",
       "seq_lru.hip")

# scalar fp32 code only: the compiler must not form packed-fp32 VALU ops
HIPCC_FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def ext(name, files, libraries=()):
    return CUDAExtension(
        name=name, sources=[os.path.join(CSRC, f) for f in files],
        libraries=list(libraries),
        extra_compile_args={"cxx": ["-O3", "-std=c++17"],
                            "nvcc": list(HIPCC_FLAGS)})


which = os.environ.get("POLYRL_EXT", "all")
modules = []
if which in ("all", "core"):
    modules.append(ext("polyrl_amd._hip", CORE, ["hipblaslt"]))
if which in ("all", "seq"):
    modules.append(ext("polyrl_amd._hip_seq", SEQ))

setup(
    name="polyrl_amd_hip",
    ext_modules=modules,
    cmdclass={"build_ext": BuildExtension.with_options(no_python_abi_suffix=False)},
)
