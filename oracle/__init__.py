"""CPU oracle for causal FlashAttention-2 parity checks.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory: it exists so that tests, the smoke check and the benchmark's CPU
baseline leg can compare the HIP kernels with a plain restatement of the
reference's naive causal attention.
"""
