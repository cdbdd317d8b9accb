"""CPU oracle for the Sarathi-Serve op library.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's ``cpu_baseline`` leg may import
this package; the shipped ops never do.

``c_oracle``            ctypes front end of the plain-C restatement
                        (``sarathi_ops_oracle.c``) that simulates the reference
                        kernels' arithmetic, rounding points included.
``torch_formulations``  the same ops written as ordinary CPU PyTorch tensor
                        code; used as an independent cross-check of the C file
                        and as the multi-threaded CPU baseline.
"""
