"""In-tree build of the megatron_amd CDNA4 HIP extension.

    PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace

Builds megatron_amd/ops/_hip_ops.so next to the package sources so the
gpurun snapshot carries the binary (no site-packages install, no JIT cache).
"""

import os

os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")

from setuptools import setup
from torch.utils.cpp_extension import BuildExtension, CppExtension, CUDAExtension

SRC = [
    "megatron_amd/ops/csrc/bindings.cpp",
    "megatron_amd/ops/csrc/rmsnorm.hip",
    "megatron_amd/ops/csrc/swiglu.hip",
    "megatron_amd/ops/csrc/rope.hip",
    "megatron_amd/ops/csrc/adamw.hip",
    "megatron_amd/ops/csrc/wgrad.hip",
    "megatron_amd/ops/csrc/cross_entropy.hip",
    "megatron_amd/ops/csrc/grouped_gemm.cpp",
    "megatron_amd/ops/csrc/causal_conv1d.hip",
    "megatron_amd/ops/csrc/attention_fwd.hip",
    "megatron_amd/ops/csrc/attention_bwd.hip",
    "megatron_amd/ops/csrc/symm_allreduce.hip",
]

# hipcc must not form packed-fp32 VALU ops on this hardware pool
HIPCC_FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

RAGGED_SRC = [
    "megatron_amd/ops/csrc/ragged/bindings.cpp",
    "megatron_amd/ops/csrc/ragged/streams.hip",
    "megatron_amd/ops/csrc/ragged/recurrent.hip",
    "megatron_amd/ops/csrc/ragged/latent_attention.hip",
    "megatron_amd/ops/csrc/ragged/latent_attention_mfma.hip",
]

HYBRID_SRC = [
    "megatron_amd/ops/csrc/hybrid/bindings.cpp",
    "megatron_amd/ops/csrc/hybrid/rows.hip",
    "megatron_amd/ops/csrc/hybrid/experts.hip",
    "megatron_amd/ops/csrc/hybrid/window_attention.hip",
    "megatron_amd/ops/csrc/hybrid/window_attention_mfma.hip",
    "megatron_amd/ops/csrc/hybrid/delta_rule.hip",
]

# the talking-heads models' extension carries the kernels it shares with the
# other two through their sources, so a fresh checkout of such a model compiles
# this extension alone
TALKING_SRC = [
    "megatron_amd/ops/csrc/talking/bindings.cpp",
    "megatron_amd/ops/csrc/talking/depth_norm.hip",
    "megatron_amd/ops/csrc/talking/talking_attention.hip",
    "megatron_amd/ops/csrc/talking/talking_attention_mfma.hip",
    "megatron_amd/ops/csrc/hybrid/rows.hip",
    "megatron_amd/ops/csrc/hybrid/experts.hip",
    "megatron_amd/ops/csrc/ragged/recurrent.hip",
]

# the extension of the models with norms on both sides of a sublayer, gated softcap attention
# and differential attention; it carries the row and expert kernels it shares with the hybrid
# extension through their sources
GATED_SRC = [
    "megatron_amd/ops/csrc/gated/bindings.cpp",
    "megatron_amd/ops/csrc/gated/sandwich_norm.hip",
    "megatron_amd/ops/csrc/gated/rope_store.hip",
    "megatron_amd/ops/csrc/gated/map_attention.hip",
    "megatron_amd/ops/csrc/gated/map_attention_mfma.hip",
    "megatron_amd/ops/csrc/hybrid/rows.hip",
    "megatron_amd/ops/csrc/hybrid/experts.hip",
]

# MEGATRON_AMD_ONLY_EXT=ragged builds just the serving kernels of the
# ragged-batch models (what a fresh checkout compiles on first use); "hybrid"
# likewise for the models built on the hybrid kernels
ONLY = os.environ.get("MEGATRON_AMD_ONLY_EXT", "")

EXTS = {
    "hip": lambda:
        CUDAExtension(
            name="megatron_amd.ops._hip_ops",
            sources=SRC,
            extra_compile_args={
                "cxx": ["-O3", "-std=c++17"],
                "nvcc": HIPCC_FLAGS + os.environ.get("MEGATRON_AMD_HIPCC_EXTRA", "").split(),
            },
            libraries=["rocblas", "hipblaslt"],
        ),
    "ragged": lambda:
        CUDAExtension(
            name="megatron_amd.ops._ragged_ops",
            sources=RAGGED_SRC,
            extra_compile_args={"cxx": ["-O3", "-std=c++17"], "nvcc": HIPCC_FLAGS},
        ),
    "hybrid": lambda:
        CUDAExtension(
            name="megatron_amd.ops._hybrid_ops",
            sources=HYBRID_SRC,
            extra_compile_args={"cxx": ["-O3", "-std=c++17"], "nvcc": HIPCC_FLAGS},
        ),
    "talking": lambda:
        CUDAExtension(
            name="megatron_amd.ops._talking_ops",
            sources=TALKING_SRC,
            extra_compile_args={"cxx": ["-O3", "-std=c++17"], "nvcc": HIPCC_FLAGS},
        ),
    "gated": lambda:
        CUDAExtension(
            name="megatron_amd.ops._gated_ops",
            sources=GATED_SRC,
            extra_compile_args={"cxx": ["-O3", "-std=c++17"], "nvcc": HIPCC_FLAGS},
        ),
    "data": lambda:
        CppExtension(
            name="megatron_amd.datasets._data_helpers",
            sources=["megatron_amd/datasets/csrc/data_helpers.cpp"],
            extra_compile_args={"cxx": ["-O3", "-std=c++17"]},
        ),
}

setup(
    name="megatron_amd_hip_ops",
    ext_modules=[make() for key, make in EXTS.items() if not ONLY or key in ONLY.split(",")],
    cmdclass={"build_ext": BuildExtension.with_options(use_ninja=True)},
)
