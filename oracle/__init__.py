"""CPU oracle (test infrastructure only).

ctypes front end of ``oracle/liboracle.so`` (built from ``oracle/cpu_reference.c`` by
``oracle/Makefile``).  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this package; the shipped library
never does.
"""
from .cpu_reference import *  # noqa: F401,F403
