"""pip install . / python setup.py build_ext --inplace: builds flex_block_attn_amd/csrc/libfba_gfx950.so with hipcc (the
recipe lives in flex_block_attn_amd/build.py) and installs the two packages, flex_block_attn_amd and its import-name
alias flex_block_attn.  No torch extension machinery is involved: the library is a plain C-ABI shared object."""
import os
import sys

from setuptools import Command, find_packages, setup
from setuptools.command.build_py import build_py

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def _build_library():
    from flex_block_attn_amd import build

    return build.build_library()


class BuildLibrary(Command):
    description = "compile the gfx950 shared library in-tree"
    user_options = [("inplace", "i", "accepted for compatibility; the library is always built in-tree")]

    def initialize_options(self):
        self.inplace = False

    def finalize_options(self):
        pass

    def run(self):
        print("built", _build_library())


class BuildPyWithLibrary(build_py):
    def run(self):
        _build_library()
        super().run()


setup(
    name="flex_block_attn_amd",
    version="1.0.0",
    description="Block-sparse attention for AMD MI355X (gfx950) with the flex-block-attn operator API",
    packages=find_packages(include=["flex_block_attn_amd", "flex_block_attn"]),
    package_data={"flex_block_attn_amd": ["csrc/*.so", "csrc/*.hip", "csrc/*.h"]},
    python_requires=">=3.9",
    cmdclass={"build_ext": BuildLibrary, "build_py": BuildPyWithLibrary},
)
