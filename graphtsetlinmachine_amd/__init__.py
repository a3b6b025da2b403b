"""MI355X-native Graph Tsetlin Machine engine (hot path only).

``Graphs`` builds the bit-packed datasets; ``MultiClassGraphTsetlinMachine``
drives the HIP kernels in ``csrc/`` through the C-ABI declared in
``include/gtm_abi.h``.
"""

from .graphs import Graphs, GraphsError  # noqa: F401


def __getattr__(name):
    # The model classes need the HIP library and torch; load them on demand so
    # that building datasets works without either.
    if name in (
        "MultiClassGraphTsetlinMachine",
        "MultiOutputGraphTsetlinMachine",
        "GraphTsetlinMachine",
        "CommonTsetlinMachine",
    ):
        from . import tm

        return getattr(tm, name)
    raise AttributeError(name)
