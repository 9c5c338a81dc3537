"""`pip install -e .` builds spear_amd/libspear_btp.so with hipcc for gfx950 and installs the
pure-Python package around it. There is no CUDA path and no architecture detection."""

import os
import sys

from setuptools import find_packages, setup
from setuptools.command.build_py import build_py

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


class BuildWithHip(build_py):
    def run(self):
        from spear_amd.csrc import build as hip_build

        print("building", hip_build.build(verbose=True))
        super().run()


setup(
    name="spear-amd",
    version="0.1.0",
    description="SPEAR Block Two-Pass kernels and Phalanx layer for AMD MI355X (gfx950)",
    packages=find_packages(include=["spear_amd", "spear_amd.*"]),
    package_data={"spear_amd": ["libspear_btp.so", "csrc/*.hip", "csrc/*.h"]},
    python_requires=">=3.10",
    install_requires=["torch>=2.0.0"],
    cmdclass={"build_py": BuildWithHip},
)
