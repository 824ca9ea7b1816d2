"""CPU oracle for the teacher-student step kernels.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this; only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may call it,
and there only as the checker (or as the timed CPU baseline), never as the
thing shipped.

Contents:
  ts_oracle.py   eager-PyTorch-on-CPU restatement of every reference function
                 on the path, each citing the reference lines it follows.  The
                 reference's arithmetic *is* a chain of PyTorch calls, so the
                 same calls on CPU tensors are its most literal restatement.
  ema_ref.c      plain-C restatement of the EMA and of the dim-0 concatenation
                 (built by the Makefile into _build/libts_oracle.so), used to
                 cross-check the PyTorch restatement bit for bit.

How each function is pinned (tests/test_oracle_*.py): fp64 closed forms written
independently in numpy, brute-force loops on tiny inputs, finite differences,
algebraic invariants and special cases, the C restatement, and structural
fixtures under tests/golden/.  The reference ships no tests, golden vectors or
fixtures for this path, so none could be used.
"""
