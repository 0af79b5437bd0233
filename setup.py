"""Build the dynamo_amd native extensions in-tree (gfx950 / MI355X only).

Usage:  PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace
The built .so files land inside dynamo_amd/ so they travel with the repo
snapshot to GPU boxes (JIT caches under ~/.cache do not).
"""
import os
import sys

os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")

from setuptools import setup  # noqa: E402
from torch.utils.cpp_extension import BuildExtension, CppExtension, CUDAExtension  # noqa: E402

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "dynamo_amd", "csrc")

hip_sources = [
    os.path.join(CSRC, f)
    for f in (
        "bindings.cpp",
        "norm.hip",
        "rope.hip",
        "activation.hip",
        "cache.hip",
        "attention_decode.hip",
        "attention_prefill.hip",
        "sampling.hip",
        "moe.hip",
        "ipc.hip",
        "probe.hip",
    )
]

SEQ = os.path.join(CSRC, "seqmix")
seq_sources = [
    os.path.join(SEQ, f)
    for f in ("seq_bindings.cpp", "seq_elementwise.hip", "seq_recurrence.hip",
              "seq_attention.hip", "seq_attention_mfma.hip", "seq_layer.hip",
              "seq_gated.hip", "seq_stream.hip")
]

# hipcc emits packed-fp32 VALU ops from plain float code unless told not to
HIPCC_FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

ext_modules = [
    CUDAExtension(
        name="dynamo_amd._hip",
        sources=hip_sources,
        extra_compile_args={
            "cxx": ["-O3", "-std=c++17"],
            "nvcc": HIPCC_FLAGS,
        },
    ),
    # recurrent / biased-attention mixers: a separate module so a model that
    # needs only these builds without the MFMA attention kernels
    CUDAExtension(
        name="dynamo_amd._hip_seq",
        sources=seq_sources,
        extra_compile_args={
            "cxx": ["-O3", "-std=c++17"],
            "nvcc": HIPCC_FLAGS,
        },
    ),
    CppExtension(
        name="dynamo_amd._core",
        sources=[os.path.join(CSRC, "core", "core.cpp")],
        extra_compile_args=["-O3", "-std=c++17"],
    ),
]

# DYNAMO_AMD_EXTS=_core,_hip_seq builds a subset (first-use builds of one
# model family); unset builds everything
_only = [e for e in os.environ.get("DYNAMO_AMD_EXTS", "").split(",") if e]
if _only:
    ext_modules = [e for e in ext_modules if e.name.split(".")[-1] in _only]

setup(
    name="dynamo_amd",
    version="0.1.0",
    packages=["dynamo_amd"],
    ext_modules=ext_modules,
    cmdclass={"build_ext": BuildExtension.with_options(use_ninja=True)},
)
