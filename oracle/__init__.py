"""CPU checkers for the banded matmul path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this module.  It is used by ``tests/``,
by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``.

Three independent statements of the same mathematics live here:

* ``cpu_oracle``   -- ctypes wrapper around ``window_matmul_oracle.c``, the
  loop-for-loop restatement of the reference's scalar CPU kernels
  (reference csrc/window_matmul/cpu/window_matmul_cpu.cpp:35-46, 83-97,
  129-141, 177-191).
* ``dense_oracle`` -- dense masked matmul in float64 (``bmm`` then gather /
  scatter then ``bmm``), a different formulation used to pin the restatement.
* ``softmax_oracle`` -- float64 numpy softmax over the band dimension (the torch step
  the reference's callers put between the two ops), for the band softmax kernels.
* ``attention_oracle`` -- the callers' chain window_matmul -> softmax -> unwindow_matmul
  composed from the two above, for the fused attention kernels.
* ``reference_module`` -- the reference's own CPU path compiled from its
  sources into ``oracle/_ref`` (only where that build exists).
"""
from .cpu_oracle import (  # noqa: F401
    load_oracle_library,
    window_matmul_forward,
    window_matmul_backward,
    unwindow_matmul_forward,
    unwindow_matmul_backward,
)
from .dense_oracle import (  # noqa: F401
    band_mask,
    dense_window_matmul,
    dense_unwindow_matmul,
    dense_window_matmul_backward,
    dense_unwindow_matmul_backward,
    band_to_dense,
    dense_to_band,
)
from .reference_module import reference_module  # noqa: F401
from . import softmax_oracle  # noqa: F401
from . import attention_oracle  # noqa: F401
