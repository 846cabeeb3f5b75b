"""CPU oracle for the per-rank data path of tccl's collectives.

TEST INFRASTRUCTURE ONLY.  Nothing under ``tccl_amd/`` imports this package; only
``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg do, and
only as the checker.

Three independent restatements of the same contract live here so that each can pin the
others:

* ``torch_ref``  -- torch CPU tensors, explicit loop over ranks (the reference named by
  the arithmetic contract: bf16 -> fp32, rank order, one rounding).
* ``c_oracle``   -- plain C (``tccl_oracle.c``), used where torch would be too slow or
  where raw bit patterns matter.
* ``np_brute``   -- numpy integer/float32 scalar-style brute force with its own bf16
  rounding, for small inputs.
"""
