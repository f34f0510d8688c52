"""Build the in-tree gfx950 HIP kernel extensions.

    PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace

Two extension modules land next to the package so they travel with
repo snapshots without a site-packages install:

* ``gllm_amd._kernels``      the kernel families of the other models
* ``gllm_amd._kernels_seq``  the dtype-generic sequence-mixer kernels
  (layer norm over an fp32 residual, windowed sink attention,
  talking-heads attention, varlen gated delta rule) plus the grouped
  MoE GEMM, activations and skinny GEMM that the linear / MoE layers
  dispatch to — the only native code a Sudevik- or Gukirax-style model
  needs, so a fresh checkout can serve one after compiling nine files
  instead of sixteen.

``GLLM_EXT=seq`` (or ``core``) restricts the build to one module.
"""

import os

os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")

from setuptools import setup
from torch.utils.cpp_extension import BuildExtension, CUDAExtension

CSRC = os.path.join("gllm_amd", "ops", "csrc")

# -packed-fp32-ops: keep hipcc from forming v_pk_*_f32 out of scalar
# float code (those forms have produced silent wrong results on gfx950)
HIP_FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
CXX_FLAGS = ["-O3", "-std=c++17"]

SEQ_SOURCES = ["bindings_seq.cpp", "layernorm.hip", "hyper.hip",
               "mingru.hip", "attention_window.hip",
               "attention_talking.hip",
               "attention_prefill.hip", "attention_decode.hip",
               "delta_rule.hip", "moe.hip", "elementwise.hip",
               "skinny_gemm.hip"]
CORE_SOURCES = ["bindings.cpp", "norm.hip", "elementwise.hip",
                "attention_decode.hip", "attention_prefill.hip",
                "attention_mla.hip", "moe.hip", "fp8.hip", "gdn.hip",
                "int4.hip", "skinny_gemm.hip", "sampling.hip",
                "custom_ar.hip"]


def _ext(name, sources):
    return CUDAExtension(
        name=name,
        sources=[os.path.join(CSRC, s) for s in sources],
        extra_compile_args={"cxx": CXX_FLAGS, "nvcc": HIP_FLAGS})


which = os.environ.get("GLLM_EXT", "all")
exts = []
if which in ("all", "core"):
    exts.append(_ext("gllm_amd._kernels", CORE_SOURCES))
if which in ("all", "seq"):
    exts.append(_ext("gllm_amd._kernels_seq", SEQ_SOURCES))

setup(
    name="gllm_amd",
    version="0.1.0",
    packages=["gllm_amd"],
    ext_modules=exts,
    cmdclass={"build_ext": BuildExtension},
)
