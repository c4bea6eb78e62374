"""CPU oracle for the FP8 / MX quantization path.  TEST INFRASTRUCTURE ONLY.

Two independent restatements live here:

* ``oracle.c_oracle``  -- ctypes binding of ``dt_oracle.c`` (bit-level C, no torch float8).
* ``oracle.eager``     -- the eager-PyTorch formulation the reference's tests compare with.

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this package;
the product (``driss_torch_amd``) never does.
"""
