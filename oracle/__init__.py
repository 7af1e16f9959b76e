"""CPU oracle for the Float8Linear hot path -- TEST INFRASTRUCTURE ONLY.

Two independent restatements of the reference's arithmetic live here:

* ``f8_oracle.c`` / :mod:`oracle.c_oracle` -- scalar C with every rounding
  spelled out (no torch involved in the arithmetic);
* :mod:`oracle.torch_oracle` -- the same composition of torch CPU operators the
  reference uses, written as plain functions.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package, and only as the checker.  The shipped
package ``float8_experimental_amd`` never does.
"""
