"""CPU oracle for the contextual-sparsity decode path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``dejavu_amd/`` may import this
package: it exists so that tests, the smoke check and the benchmark's
``cpu_baseline`` leg have an independent statement of what the HIP kernels
must compute.
"""
