"""Builds and installs the drop-in names: ``fast_rnnt`` (alias package), top-level
``_fast_rnnt`` (operator module) and ``fast_rnnt_amd`` (the implementation with its gfx950
library and its compiled torch operator module).

Counterpart of the reference's setup.py: there ``build_ext`` drives CMake for ``_fast_rnnt``
(setup.py:48-54) and the package is installed beside it (:97-125); here ``build_py`` runs
``make -C fast_rnnt_amd/csrc`` (hipcc for libfast_rnnt_amd.so, g++ against the installed
torch for fast_rnnt_amd/_C*.so) and the results travel as package data.  Needs /opt/rocm
(hipcc) and the torch the module will be used with; no network.
"""
import glob
import os
import re
import subprocess

import setuptools
from setuptools.command.build_py import build_py

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "fast_rnnt_amd", "csrc")


def version():
    text = open(os.path.join(HERE, "fast_rnnt_amd", "__init__.py")).read()
    return re.search(r'__version__ = "([^"]+)"', text).group(1)


class BuildNativeThenPy(build_py):
    """Compile the native pieces in-tree (make only rebuilds what is out of date), then
    collect the Python files and, as package data, what make produced."""

    def run(self):
        jobs = os.environ.get("MAX_JOBS", "8")
        print(f"building the gfx950 library and the torch operator module: make -C {CSRC} -j{jobs}")
        subprocess.check_call(["make", "-C", CSRC, f"-j{jobs}", "-s"])
        built = [os.path.join(CSRC, "libfast_rnnt_amd.so")] + glob.glob(
            os.path.join(HERE, "fast_rnnt_amd", "_C*.so"))
        missing = [p for p in built[:1] if not os.path.exists(p)]
        if missing or len(built) < 2:
            raise RuntimeError(f"make did not produce {missing or 'fast_rnnt_amd/_C*.so'}")
        super().run()


setuptools.setup(
    name="fast_rnnt",
    version=version(),
    description="fast_rnnt's RNN-T loss hot path on AMD MI355X (gfx950)",
    packages=["fast_rnnt", "fast_rnnt_amd"],
    py_modules=["_fast_rnnt"],
    package_data={"fast_rnnt_amd": ["csrc/libfast_rnnt_amd.so", "_C*.so"]},
    data_files=[("include", ["include/fast_rnnt_amd.h"])],
    install_requires=["torch"],
    cmdclass={"build_py": BuildNativeThenPy},
    zip_safe=False,
)
