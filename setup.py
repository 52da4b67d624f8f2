"""pip install . — builds the gfx950 library and its torch binding with the in-tree Makefile
(hipcc from ROCm and g++ against the installed torch must be present) and installs the
``ds_splat`` / ``ds_splat_amd`` packages with the two shared objects as package data.
It plays the role of the reference's setup.py (a torch CUDAExtension build); there is no
hipify step and no CUDA source here.
"""
import os
import subprocess

from setuptools import setup
from setuptools.command.build_py import build_py

ROOT = os.path.dirname(os.path.abspath(__file__))


class BuildNative(build_py):
    def run(self):
        jobs = str(min(16, os.cpu_count() or 1))
        subprocess.run(["make", "-C", os.path.join(ROOT, "ds_splat_amd", "csrc"), "-j", jobs], check=True)
        super().run()


setup(
    name="ds_splat_amd",
    version="1.0.0",
    description="MI355X (gfx950) native 3D Gaussian Splatting rasterizer with the ds_splat API",
    packages=["ds_splat", "ds_splat_amd"],
    package_data={"ds_splat_amd": ["lib/libdsx.so", "lib/_dsx_torch*.so"]},
    include_package_data=False,
    python_requires=">=3.9",
    install_requires=[],  # torch (ROCm build) must already be installed: the binding links against it
    cmdclass={"build_py": BuildNative},
    zip_safe=False,
)
