"""Build the gfx950 extension in place:  python setup.py build_ext --inplace

Counterpart of the reference's setup.py (:29-48), for one target only: AMD MI355X (gfx950).
There is no CUDA path and no source translation step; `buildlib.py` hands csrc/*.hip to hipcc and
csrc/binding.cpp to the host compiler.  The artefacts (libsma_hip.so and the sparse_attn_cuda
module) are written next to this file.
"""
import os
import sys

from setuptools import Command, setup

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import buildlib  # noqa: E402


class build_ext(Command):
    description = "compile libsma_hip.so (hipcc, gfx950) and the sparse_attn_cuda module in place"
    user_options = [("inplace", "i", "accepted for familiarity; the build is always in place")]

    def initialize_options(self):
        self.inplace = True

    def finalize_options(self):
        pass

    def run(self):
        buildlib.build_all()


setup(
    name="sparse_mask_attention_amd",
    version="0.1.0",
    description="Sparse-mask attention for AMD MI355X (gfx950): hand-written HIP kernels",
    packages=[],
    cmdclass={"build_ext": build_ext},
    python_requires=">=3.8",
)
