"""CPU oracle for the AdderNet convolution hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
package: it exists so that tests, the smoke check and the CPU-baseline leg of
the benchmark can check the HIP kernels against an independent restatement of
the reference's arithmetic.
"""
