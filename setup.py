"""Build the parallax_amd HIP extension in-tree for gfx950 (MI355X).

    PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace

The built .so files land at parallax_amd/ops/_C.*.so (attention, GEMM, MoE,
sampler kernels) and parallax_amd/ops/_mix.*.so (sequence mixers: fp32-residual
layer norm, sliding-window latent attention, gated linear attention, sandwich
RMS norm, row-cache attention, post-norm residual step, minGRU). Both are
git-ignored; they travel to the GPU box with the gpurun snapshot.
PARALLAX_EXT=_mix (or _C) builds one of them only.
"""

import os

from setuptools import setup
from torch.utils.cpp_extension import BuildExtension, CUDAExtension

os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "parallax_amd", "ops", "csrc")

sources = [
    os.path.join(CSRC, "bindings.cpp"),
    os.path.join(CSRC, "lt_gemm.cpp"),
    os.path.join(CSRC, "elementwise.hip"),
    os.path.join(CSRC, "paged_attention.hip"),
    os.path.join(CSRC, "paged_attention_mfma.hip"),
    os.path.join(CSRC, "mla_attention.hip"),
    os.path.join(CSRC, "prefill_attention.hip"),
    os.path.join(CSRC, "moe.hip"),
    os.path.join(CSRC, "skinny_gemm.hip"),
    os.path.join(CSRC, "indexer.hip"),
    os.path.join(CSRC, "sampler.hip"),
]
sources = [s for s in sources if os.path.exists(s)]

# hipcc -O3 turns plain float code into packed-fp32 instructions; every kernel
# here keeps its fp32 operations scalar (-packed-fp32-ops)
HIP_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
MIX_HIP_FLAGS = HIP_FLAGS

mix_sources = [
    os.path.join(CSRC, "mix_bindings.cpp"),
    os.path.join(CSRC, "layernorm.hip"),
    os.path.join(CSRC, "latent_attention.hip"),
    os.path.join(CSRC, "gla.hip"),
    os.path.join(CSRC, "sandwich_norm.hip"),
    os.path.join(CSRC, "row_attention.hip"),
    os.path.join(CSRC, "row_attention_mfma.hip"),
    os.path.join(CSRC, "post_norm.hip"),
    os.path.join(CSRC, "group_norm.hip"),
]

wanted = [x for x in os.environ.get("PARALLAX_EXT", "_C,_mix").split(",") if x]
extensions = []
if "_C" in wanted:
    extensions.append(
        CUDAExtension(
            name="parallax_amd.ops._C",
            sources=sources,
            libraries=["hipblaslt"],
            extra_compile_args={"cxx": ["-O3", "-std=c++17"], "nvcc": HIP_FLAGS},
        )
    )
if "_mix" in wanted:
    extensions.append(
        CUDAExtension(
            name="parallax_amd.ops._mix",
            sources=mix_sources,
            extra_compile_args={"cxx": ["-O3", "-std=c++17"],
                                "nvcc": MIX_HIP_FLAGS},
        )
    )

setup(
    name="parallax_amd_ext",
    entry_points={
        "console_scripts": ["parallax_amd = parallax_amd.cli:main"],
    },
    ext_modules=extensions,
    cmdclass={"build_ext": BuildExtension.with_options(use_ninja=True)},
)
