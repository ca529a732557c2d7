"""Build and install the MI355X inpainting layers.

`python setup.py build_ext --inplace` (or `install`) compiles the HIP library for gfx950 with hipcc
into customnetworklayers_amd/libinpaint_hip.so; the Python modules bind it through its C ABI
(include/*.h), with ctypes and, for the two inpainting layers, also as compiled PyTorch extensions
(customnetworklayers_amd/cudaTV/tvInpaint_hip_ext.so, cudaTGV/tgvInpaint_hip_ext.so).  The reference builds one torch CUDAExtension per layer
(cudaTV/setup.py:16-28, cudaTGV/setup.py:16-29, cudaQuadFit/setup.py:16-28, cudaMedian/setup.py:16-27 of the
reference); the module names it produces -- tvInpaint_cuda_ext, tgvInpaint_cuda_ext, QuadFit_cuda_ext,
median_cuda_ext -- are kept as importable top-level modules.
"""
import os
import subprocess

from setuptools import Command, setup
from setuptools.command.build_py import build_py

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "customnetworklayers_amd", "csrc")


class BuildHip(Command):
    description = "compile the HIP library for gfx950"
    user_options = [("inplace", "i", "kept for compatibility: the library is always built in-tree")]

    def initialize_options(self):
        self.inplace = 1

    def finalize_options(self):
        pass

    def run(self):
        subprocess.check_call(["make", "-C", CSRC, "-j8", "all"])
        # the compiled PyTorch bindings over the C ABI (host C++; the ctypes bindings need none of this)
        subprocess.check_call(["make", "-C", CSRC, "-j8", "bindings"])


class BuildPyWithHip(build_py):
    def run(self):
        self.run_command("build_ext")
        super().run()


setup(
    name="customnetworklayers_amd",
    version="0.1.0",
    description="TV / TGV FISTA inpainting layers, quadratic fit and histogram median for MI355X (gfx950)",
    packages=["customnetworklayers_amd", "customnetworklayers_amd.cudaTV", "customnetworklayers_amd.cudaTGV",
              "customnetworklayers_amd.cudaQuadFit", "customnetworklayers_amd.cudaMedian"],
    package_data={"customnetworklayers_amd": ["libinpaint_hip.so"], "customnetworklayers_amd.cudaTV": ["tvInpaint_hip_ext.so"],
                  "customnetworklayers_amd.cudaTGV": ["tgvInpaint_hip_ext.so"]},
    py_modules=["tvInpaint_cuda_ext", "tgvInpaint_cuda_ext", "QuadFit_cuda_ext", "median_cuda_ext", "TVInpainting",
                "TGVInpainting", "QuadFitting", "median"],
    cmdclass={"build_ext": BuildHip, "build_py": BuildPyWithHip},
)
