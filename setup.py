"""In-tree build of the MI355X-native extensions.

Usage:  PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace

Two extensions:
  xllm_service_amd._ops   HIP/CDNA4 kernels (gfx950) + torch bindings
  (the pure-C++ control-plane core lives in _core; added as it lands)
"""
import os

from setuptools import setup

os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")

from torch.utils.cpp_extension import BuildExtension, CUDAExtension  # noqa: E402

ROOT = os.path.dirname(os.path.abspath(__file__))
OPS = os.path.join(ROOT, "xllm_service_amd", "csrc", "ops")
HYB = os.path.join(ROOT, "xllm_service_amd", "csrc", "hybrid")

# hipcc only: fp32 math compiles to scalar-lane ops (no packed fp32 forms)
HIP_FLAGS = ["-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops"]

ext_modules = [
    CUDAExtension(
        name="xllm_service_amd._ops",
        sources=[
            os.path.join(OPS, f)
            for f in (
                "bindings.cpp",
                "norm.hip",
                "rope.hip",
                "activation.hip",
                "cache.hip",
                "paged_attn_decode.hip",
                "paged_attn_prefill.hip",
                "sampling.hip",
                "gemm.hip",
                "skinny_gemm.hip",
                "packed_gemm.hip",
            )
        ],
        extra_compile_args={
            "cxx": ["-O3", "-std=c++17"],
            "nvcc": HIP_FLAGS,
        },
    ),
    # hybrid sequence mixers (latent attention, decayed and gated linear
    # recurrences, the gated delta rule, soft-capped / windowed paged attention,
    # short convolutions, rotary turns with head norms), grouped and post
    # norms, PolyNorm, residual streams and routed experts; bf16 and fp32
    # activations
    CUDAExtension(
        name="xllm_service_amd._ops_hybrid",
        sources=[
            os.path.join(HYB, f)
            for f in ("bindings.cpp", "norms.hip", "latent_attn.hip",
                      "latent_attn_mfma.hip", "decay_attn.hip", "moe.hip",
                      "streams.hip", "short_conv.hip",
                      "gated_recurrence.hip", "capped_attn.hip",
                      "capped_attn_mfma.hip", "rownorm_rope.hip",
                      "delta_rule.hip", "rope_headnorm.hip")
        ],
        extra_compile_args={
            "cxx": ["-O3", "-std=c++17"],
            "nvcc": HIP_FLAGS,
        },
    ),
]

# XLLM_BUILD_EXT=<module name>[,<module name>] builds only those extensions
# (a worker compiles just what its model needs on first start)
_only = [n for n in os.environ.get("XLLM_BUILD_EXT", "").split(",") if n]
if _only:
    ext_modules = [e for e in ext_modules
                   if e.name.rsplit(".", 1)[-1] in _only]

setup(
    name="xllm_service_amd",
    version="0.1.0",
    packages=["xllm_service_amd"],
    ext_modules=ext_modules,
    cmdclass={"build_ext": BuildExtension},
)
