"""CPU oracle for the batched radix-2 C2C FFT path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this directory.  It is used by
``tests/``, by ``__graft_entry__.smoke()`` as the checker and by ``bench.py``
for the timed CPU baseline leg -- never as a compute fallback.
"""
