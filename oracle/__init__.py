"""CPU oracle for the W8A8 fp8 linear path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the shipped ``phyai_amd`` package never
does.  Two independent statements of the same arithmetic live here:

* :mod:`oracle.ref`   - the reference's tensor expressions written with torch
  CPU ops (``torch`` is a library both sides share, not the reference).
* :mod:`oracle.cport` - ctypes bindings of ``fp8_oracle.c``, a plain-C
  restatement that does not depend on torch's casts at all.

The tests cross-check the two against each other, against closed forms and
against the committed fixtures under ``tests/golden/``.
"""
