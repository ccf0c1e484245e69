#!/usr/bin/env python3
"""Packaging of transducer_amd: ``python setup.py build_ext --inplace`` (or an editable install
with ``--no-build-isolation``) compiles the three native libraries in-tree with hipcc and g++.

Plays the part of the reference's setup.py:23-73 (a build_ext that shells out to CMake, which in
turn fetches pybind11 from the network, cmake/Buildpybind11.cmake:4-5): here the build_ext runs
transducer_amd/build.py, which needs hipcc, g++ and the installed pybind11 headers and nothing
from the network.
"""
import importlib.util
import os

from setuptools import Extension, setup
from setuptools.command.build_ext import build_ext

__version__ = "0.1.0"
HERE = os.path.dirname(os.path.abspath(__file__))


def _load_build_module():
    # by path: importing the package itself would want the libraries that are about to be built
    spec = importlib.util.spec_from_file_location(
        "_transducer_amd_build", os.path.join(HERE, "transducer_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


class HipBuild(build_ext):
    """Builds librnnt_hip.so, libtransducer.so and the _transducer module: next to the sources
    with --inplace, else straight into build_lib (objects into build_temp), leaving the source
    tree untouched."""

    def run(self):
        build = _load_build_module()
        if self.inplace:
            build.build_all()
        else:
            build.build_all(out_dir=os.path.join(self.build_lib, "transducer_amd"),
                            obj_dir=os.path.join(self.build_temp, "transducer_amd"))

    def get_outputs(self):
        return []


setup(
    name="transducer_amd",
    version=__version__,
    description="RNN transducer loss and viterbi path for MI355X (gfx950), behind the API of "
                "awni/transducer",
    packages=["transducer_amd"],
    package_data={"transducer_amd": ["*.so", "csrc/*.hip", "csrc/*.h", "csrc/*.cpp"]},
    ext_modules=[Extension("transducer_amd._transducer", sources=[])],
    cmdclass={"build_ext": HipBuild},
    zip_safe=False,
    python_requires=">=3.8",
)
