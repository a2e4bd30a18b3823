"""TEST INFRASTRUCTURE ONLY: CPU oracle of the D2Conv3D operator path.

`oracle.cpu` wraps the C restatement (libd2c_oracle.so, built by
oracle/Makefile) for torch CPU tensors; `oracle.brute` is an independent
pure-Python loop restatement of the reference test-suite's own expected_fn
(ops/dconv-native/test/test_deform_conv.py:127-191) used to pin the C oracle
on tiny inputs.  Only tests, the smoke check and the benchmark's CPU-baseline
leg import this package.
"""
