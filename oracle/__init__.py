"""CPU oracle for the Mixture-of-Experts hot path.

TEST INFRASTRUCTURE ONLY. Nothing in the product package may import this
package; it exists so that tests, the smoke check and the CPU-baseline leg of
the benchmark have an independent statement of the algorithm to compare the
HIP path against.
"""
