"""Loader for ``oracle/_ref`` (TEST INFRASTRUCTURE ONLY).

``oracle/_ref/_fast_rnnt*.so`` is the reference's own CPU operator module
(fast_rnnt/python/csrc/fast_rnnt.cu:24), compiled from the reference sources by
``make -C oracle ref``.  It is git-ignored; when it has not been built,
``load()`` returns None and the tests that cross-check the plain-C restatement
against it are skipped.
"""
import glob
import importlib.util
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_REF_DIR = os.path.join(_HERE, "_ref")
_module = None


def build(reference_root: str = "/root/reference") -> bool:
    """Run the reference recipe if the reference tree is present."""
    if not os.path.isdir(reference_root):
        return False
    subprocess.check_call(["make", "-C", _HERE, "-s", "ref", f"REF={reference_root}"])
    return True


def load():
    """Return the built reference module ``_fast_rnnt`` or None."""
    global _module
    if _module is not None:
        return _module
    hits = sorted(glob.glob(os.path.join(_REF_DIR, "_fast_rnnt*.so")))
    if not hits:
        return None
    import torch  # noqa: F401  (the module links against libtorch)

    spec = importlib.util.spec_from_file_location("_fast_rnnt", hits[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    _module = mod
    return mod
