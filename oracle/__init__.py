"""CPU oracle for HSTU jagged attention.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this directory.  It is used by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` as the checker / the timed CPU reference, never as a compute path.

Contents
--------
``hstu_oracle.py``  fp32/fp64 PyTorch-on-CPU restatement of
    ``generative_recommenders/ops/pytorch/pt_hstu_attention.py`` (mask, pad,
    ``pytorch_hstu_mha``, ``pytorch_cached_hstu_mha``) plus a per-sequence form
    of the same mathematics that never builds the ``[B, H, N, N]`` tensor.
``hstu_ref.c``      an independent scalar C restatement (double accumulation,
    mask written per position class instead of via the id formula) used to pin
    the PyTorch restatement on small inputs.

How each function is pinned is listed at the top of ``hstu_oracle.py``.
"""
