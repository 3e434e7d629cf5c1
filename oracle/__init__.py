"""CPU oracle for the fused optimizer-step path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is the checker the HIP kernels are compared against, and the
thing timed as the CPU baseline.

Two independent restatements of optimi's PyTorch for-loop step live here:

* ``oracle.forloop``  – op-for-op torch restatement (the same in-place ATen
  ops in the same order), so every intermediate is rounded to the tensor dtype
  exactly where the reference rounds it.  Runs on CPU tensors.
* ``oracle/scalar_ref.c`` (loaded through ``oracle.scalar``) – a scalar C
  emulator that spells each rounding point and each fused multiply-add out by
  hand.  It carries no torch dependency and is what the HIP kernels are
  expected to equal bit for bit.

Pinning status of each function is listed at the top of ``oracle/forloop.py``.
"""
