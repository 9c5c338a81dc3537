"""`pip install -e .` builds spear_amd/libspear_btp.so and its torch binding spear_amd/_btp_ext.so with
hipcc for gfx950 and installs the Python package around them. There is no CUDA path and no architecture detection."""

import os
import sys

from setuptools import find_packages, setup
from setuptools.command.build_py import build_py

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


class BuildWithHip(build_py):
    def run(self):
        from spear_amd.csrc import build as hip_build

        print("building", hip_build.build(verbose=True))
        print("building", hip_build.build_extension(verbose=True))
        super().run()


setup(
    name="spear-amd",
    version="0.1.0",
    description="SPEAR Block Two-Pass kernels and Phalanx layer for AMD MI355X (gfx950)",
    # `spear` is the reference's import name: an alias package without code of its own
    packages=find_packages(include=["spear_amd", "spear_amd.*", "spear"]),
    package_data={"spear_amd": ["libspear_btp.so", "_btp_ext.so", "csrc/*.hip", "csrc/*.h", "csrc/*.cpp"]},
    python_requires=">=3.10",
    install_requires=["torch>=2.0.0"],
    cmdclass={"build_py": BuildWithHip},
)
