"""`python setup.py build_ext --inplace` / `install`: counterpart of the reference's setup.py
(reference setup.py:7-20, a CUDAExtension named `fused_attn`).  The device code is compiled by
hipcc for gfx950 into a C-ABI shared library and the torch binding by g++ (see
fused_attention_amd/build.py); setuptools only drives those two steps and packages the results."""
import os
import shutil

from setuptools import Extension, setup
from setuptools.command.build_ext import build_ext

HERE = os.path.dirname(os.path.abspath(__file__))


class BuildGfx950(build_ext):
    def run(self):
        import sys

        sys.path.insert(0, HERE)
        from fused_attention_amd import build as fa_build

        fa_build.build_kernel_library()
        fa_build.build_smoke_binary()
        built = fa_build.build_torch_binding()
        if not self.inplace:
            target = self.get_ext_fullpath("fused_attn")
            os.makedirs(os.path.dirname(target), exist_ok=True)
            shutil.copy(built, target)


setup(
    name="fused_attn",
    version="0.1.0",
    packages=["fused_attention_amd"],
    package_data={"fused_attention_amd": ["libfused_attn_gfx950.so", "csrc/*"]},
    ext_modules=[Extension("fused_attn", sources=[])],
    cmdclass={"build_ext": BuildGfx950},
)
