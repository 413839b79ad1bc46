"""CPU oracle for the FP8 block-scale path.  TEST INFRASTRUCTURE ONLY.

Nothing under ``aiter_amd/`` may import this package: it exists so that tests, the smoke
check and the benchmark's CPU-baseline leg can check (and time) the reference semantics on
host cores.  Two restatements live here:

* ``oracle.c_oracle``  - ctypes binding of ``libfp8bs_oracle.so`` (scalar C, bit-level)
* ``oracle.torch_ref`` - torch-CPU restatement of the reference's own torch functions
"""
