"""CPU oracle for deformable multi-view SDPA -- TEST INFRASTRUCTURE ONLY.

Nothing that ships imports this package. It is loaded by ``tests/``, by the
smoke check and by the CPU-baseline leg of ``bench.py``, and only as the
checker (or the timed CPU baseline), never as a compute path of the operator.

Two independent restatements of the reference's eager semantics
(``ops/torch.py:5-28`` forward, ``ops/triton.py:330-360,464`` backward):

* :mod:`oracle.c_oracle`   -- explicit scalar loops in C (``dsdpa_oracle.c``),
  double accumulation, per-tap bounds tests; the oracle proper.
* :mod:`oracle.torch_eager` -- the same op through the ATen library routines
  ``grid_sample`` + ``softmax`` with PyTorch autograd for the gradients; used
  to pin the C oracle and as the "host-CPU torch" baseline.
"""
from .c_oracle import oracle_fwd, oracle_bwd, oracle_taps, build_oracle  # noqa: F401
