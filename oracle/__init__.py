"""CPU checkers for the bitmap SpMM path.  TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke test and the benchmark's cpu_baseline leg import this
package; the shipped library and its host layer never do.
"""
