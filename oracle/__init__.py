"""CPU checker for the tensor hot path (test infrastructure, never shipped).

`oracle.lib` wraps oracle/libhyle_oracle.so (this repo's C restatement of the
reference's scalar semantics); `oracle.ref` wraps oracle/_ref (the reference's
own scalar floor compiled from its sources, present only where it was built).
Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package.
"""
from . import lib  # noqa: F401
