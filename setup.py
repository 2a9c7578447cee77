"""Build the gfx950 HIP kernel extension in-tree.

Usage:  PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace

The resulting _kernels .so lands inside inference_gateway_amd/ops/ so the
gpurun snapshot carries it to the GPU box (JIT caches under ~/.cache do not
travel).
"""
import os
from pathlib import Path

from setuptools import setup

os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")

from torch.utils import cpp_extension  # noqa: E402

ROOT = Path(__file__).parent
CSRC = ROOT / "inference_gateway_amd" / "ops" / "csrc"

def _hip_sources(d):
    # hipify leaves shadow copies (x_hip.hip) beside the sources
    return sorted(str(p) for p in d.glob("*.hip")
                  if not p.name.endswith("_hip.hip"))


sources = [str(CSRC / "bindings.cpp")] + _hip_sources(CSRC)
HYB = ROOT / "inference_gateway_amd" / "ops" / "csrc_hybrid"
hybrid_sources = [str(HYB / "bindings.cpp")] + _hip_sources(HYB)

REC = ROOT / "inference_gateway_amd" / "ops" / "csrc_recurrent"
# the recurrent extension also compiles the two hybrid source files whose
# row kernels (fused add + RMS norm, squared ReLU) its models share
recurrent_sources = [str(REC / "bindings.cpp")] + _hip_sources(REC) + [str(HYB / "parallel_ops.hip"), str(HYB / "hybrid_ops.hip")]

# packed-fp32 instruction selection is switched off for all device code
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _ext(name, srcs):
    return cpp_extension.CUDAExtension(
        name=name,
        sources=srcs,
        extra_compile_args={"cxx": ["-O3", "-std=c++17"],
                            "nvcc": list(HIPCC_FLAGS)},
    )


# IGW_BUILD_EXT=hybrid|kernels|recurrent builds just one extension (a
# process that serves one model family compiles only what it loads);
# default: all
_which = os.environ.get("IGW_BUILD_EXT", "all")
ext_modules = []
if _which in ("all", "kernels"):
    ext_modules.append(_ext("inference_gateway_amd.ops._kernels", sources))
if _which in ("all", "hybrid"):
    ext_modules.append(_ext("inference_gateway_amd.ops._hybrid",
                            hybrid_sources))

if _which in ("all", "recurrent"):
    ext_modules.append(_ext("inference_gateway_amd.ops._recurrent",
                            recurrent_sources))

setup(
    name="inference_gateway_amd_kernels",
    ext_modules=ext_modules,
    cmdclass={"build_ext": cpp_extension.BuildExtension},
)
