"""The host's garbage collector beside a serving loop.

A full collection walks every container object that is alive.  After a model is loaded that
is some 170,000 objects (the imported modules, the parts, the kernel bindings): 20 ms, in which
the loop issues nothing, and it comes back every few thousand allocations of the loop itself.
What the loop keeps for long (argument blocks of product calls, cached views) is therefore kept
in forms that the collector does not walk (``ops.kernels.linear``: bytes), and the entry points
freeze what is alive once the engine stands.
"""

import gc


def settle():
    """Collect once, then move everything that is alive into the permanent generation: later
    collections do not walk it again.  Objects made from now on are collected as before;
    ``gc.unfreeze()`` undoes it."""
    gc.collect()
    gc.freeze()
