"""Installs the drop-in names: ``fast_rnnt`` (alias package), top-level ``_fast_rnnt``
(operator module) and ``fast_rnnt_amd`` (the implementation with its prebuilt gfx950
library).  The library is built first, in-tree, by ``make -C fast_rnnt_amd/csrc``
(hipcc); this script only packages it.  Counterpart: the reference's setup.py:97-125.
"""
import os
import re

import setuptools

HERE = os.path.dirname(os.path.abspath(__file__))


def version():
    text = open(os.path.join(HERE, "fast_rnnt_amd", "__init__.py")).read()
    return re.search(r'__version__ = "([^"]+)"', text).group(1)


if not os.path.exists(os.path.join(HERE, "fast_rnnt_amd", "csrc", "libfast_rnnt_amd.so")):
    raise SystemExit("build the library first: make -C fast_rnnt_amd/csrc")

setuptools.setup(
    name="fast_rnnt",
    version=version(),
    description="fast_rnnt's RNN-T loss hot path on AMD MI355X (gfx950)",
    packages=["fast_rnnt", "fast_rnnt_amd"],
    py_modules=["_fast_rnnt"],
    package_data={"fast_rnnt_amd": ["csrc/libfast_rnnt_amd.so"]},
    data_files=[("include", ["include/fast_rnnt_amd.h"])],
    install_requires=["torch"],
    zip_safe=False,
)
