"""Build the sutro_amd._C HIP extension in-tree for MI355X (gfx950).

    PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace
"""

import os

os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")

from setuptools import setup
from torch.utils.cpp_extension import BuildExtension, CUDAExtension

SOURCES = [
    "csrc/bindings.cpp",
    "csrc/rmsnorm.hip",
    "csrc/elementwise.hip",
    "csrc/rope_cache.hip",
    "csrc/qkv_prep.hip",
    "csrc/pool.hip",
    "csrc/attn_decode.hip",
    "csrc/attn_decode_mfma.hip",
    "csrc/attn_prefill.hip",
    "csrc/gemm_tn.hip",
    "csrc/sampler.hip",
    "csrc/grouped_gemm.hip",
]

# kernels of layer-list decoders (local attention, gated delta rule, gated
# scalar-gain norms): an extension of their own, so a process that serves
# only such a model builds and loads only these
MIX_SOURCES = [
    "csrc/mix_bindings.cpp",
    "csrc/mix_norm.hip",
    "csrc/mix_attn.hip",
    "csrc/mix_attn_mfma.hip",
    "csrc/mix_delta.hip",
    "csrc/mix_stream.hip",
    "csrc/mix_prep.hip",
    "csrc/mix_mlstm.hip",
    "csrc/mix_moe.hip",
    "csrc/mix_prenorm.hip",
    "csrc/mix_decay.hip",
    # the matrix-core expert GEMM serves both extensions
    "csrc/grouped_gemm.hip",
]

# hipcc's automatic packed-fp32 forms are switched off for all device code
HIP_FLAGS = ["-O3", "--offload-arch=gfx950",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

EXTENSIONS = {"_C": SOURCES, "_C_mix": MIX_SOURCES}
# SUTRO_AMD_EXTENSIONS=_C_mix builds only the named extensions
_only = [n for n in os.environ.get("SUTRO_AMD_EXTENSIONS", "").split(",") if n]

setup(
    name="sutro-amd-kernels",
    ext_modules=[
        CUDAExtension(
            name="sutro_amd." + name,
            sources=srcs,
            extra_compile_args={"cxx": ["-O3"], "nvcc": list(HIP_FLAGS)},
        )
        for name, srcs in EXTENSIONS.items() if not _only or name in _only
    ],
    cmdclass={"build_ext": BuildExtension},
)
