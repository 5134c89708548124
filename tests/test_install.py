"""setup.py builds what it installs, and the installed tree works on its own (CPU only).

Counterpart: the reference's setup.py:48-54 (build_ext drives the native build) and
:97-125 (the package is installed under the name ``fast_rnnt`` beside ``_fast_rnnt``).
The install goes to a temporary directory (pip --target, no index, no build isolation) and
is imported from a process whose path holds that directory and not this repository.
"""
import os
import subprocess
import sys
import textwrap

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHECK = textwrap.dedent("""
    import os, sys
    target = sys.argv[1]
    import torch
    import fast_rnnt, _fast_rnnt, fast_rnnt_amd
    import fast_rnnt_amd.k2_compat as k2
    for mod in (fast_rnnt, _fast_rnnt, fast_rnnt_amd):
        assert os.path.realpath(mod.__file__).startswith(os.path.realpath(target)), mod.__file__
    assert fast_rnnt.__version__.startswith("1.2") and fast_rnnt.with_cuda() is True
    assert k2.rnnt_loss_pruned is fast_rnnt.rnnt_loss_pruned
    from fast_rnnt_amd import _lib
    lib = _lib.load()                      # the installed gfx950 library
    assert os.path.realpath(_lib.LIB_PATH).startswith(os.path.realpath(target))
    assert lib.frnnt_version() >= 100
    ops = _lib.ops()                       # the installed torch operator module
    assert os.path.realpath(ops.__file__).startswith(os.path.realpath(target))
    assert hasattr(torch.ops.fast_rnnt_amd, "simple_loss")
    try:                                   # argument checks run in the compiled module
        _fast_rnnt.mutual_information_forward(torch.zeros(1, 2, 4), torch.zeros(1, 3, 3), None,
                                              torch.zeros(1, 3, 4))
    except RuntimeError as err:
        assert "GPU" in str(err)
    else:
        raise SystemExit("CPU tensors were not refused")
    print("installed tree ok")
""")


def test_pip_install_to_a_fresh_directory(tmp_path):
    target = tmp_path / "site"
    env = dict(os.environ, PIP_DISABLE_PIP_VERSION_CHECK="1", PIP_NO_INDEX="1")
    pip = [sys.executable, "-m", "pip", "install", "--no-build-isolation", "--no-deps", "--no-index",
           "--quiet", "--target", str(target), ROOT]
    done = subprocess.run(pip, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=900)
    if done.returncode != 0:
        pytest.fail("pip install failed:\n" + done.stdout[-3000:])
    names = set(os.listdir(target))
    assert {"fast_rnnt", "fast_rnnt_amd", "_fast_rnnt.py"} <= names, names
    assert (target / "fast_rnnt_amd" / "csrc" / "libfast_rnnt_amd.so").exists()
    # import from there only: a clean interpreter whose path does not hold the repository
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    env["PYTHONPATH"] = str(target)
    run = subprocess.run([sys.executable, "-c", CHECK, str(target)], env=env, cwd=str(tmp_path),
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert run.returncode == 0 and "installed tree ok" in run.stdout, run.stdout[-3000:]
