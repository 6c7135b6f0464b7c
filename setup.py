"""Build the kllms_amd gfx950 HIP extension in-tree.

    PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace

Produces kllms_amd/_C*.so next to the package sources so the snapshot that
ships to a GPU box carries the built extension, then compiles the
per-family extensions (kllms_amd/ops/jit.py: _C_seq) the same way they are
compiled on demand in a checkout with nothing built.
"""

import os
import sys

from setuptools import setup

os.environ.setdefault("PYTORCH_ROCM_ARCH", "gfx950")

from torch.utils.cpp_extension import BuildExtension, CUDAExtension  # noqa: E402

HIP_DIR = os.path.join("kllms_amd", "ops", "hip")
SOURCES = [
    os.path.join(HIP_DIR, f)
    for f in (
        "bindings.hip",
        "elementwise.hip",
        "attn_decode.hip",
        "attn_prefill.hip",
        "sampling.hip",
        "mfma_selftest.hip",
        "allreduce.hip",
        "moe.hip",
        "levenshtein.hip",
    )
]

setup(
    name="kllms_amd_C",
    ext_modules=[
        CUDAExtension(
            name="kllms_amd._C",
            sources=SOURCES,
            extra_compile_args={
                "cxx": ["-O3"],
                # packed-fp32 instruction selection is switched off for all
                # device code (the host pass warns that it does not know the
                # feature; harmless)
                "nvcc": ["-O3", "--offload-arch=gfx950", "-std=c++17",
                         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"],
            },
        )
    ],
    cmdclass={"build_ext": BuildExtension},
)

if "build_ext" in sys.argv:
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from kllms_amd.ops import jit

    for _name in jit.EXTENSIONS:
        print("built", jit.build(_name))
