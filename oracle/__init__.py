"""CPU oracle for the fast_rnnt loss hot path -- TEST INFRASTRUCTURE ONLY.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package, and only as the checker.  The shipped
package ``fast_rnnt_amd`` never imports it.

Modules:
  recursion   ctypes front end of ``liboracle_mi.so`` (mi_oracle.c): the lattice
              recursion forward/backward and the autograd wrapper that mirrors
              fast_rnnt/python/fast_rnnt/mutual_information.py.
  losses      torch-CPU restatement of the px/py builders, the pruning helpers
              and the four loss wrappers of
              fast_rnnt/python/fast_rnnt/rnnt_loss.py.
  ref_build   loader for ``oracle/_ref`` (the reference's own C++ operator,
              compiled from its sources by ``make -C oracle ref``), when built.
"""
