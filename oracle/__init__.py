"""CPU oracle for the V-MoE inference MoE layer.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (``vmoe_amd``) may
import this package: it exists so that tests, the smoke check and the
``cpu_baseline`` leg of the benchmark have an independent statement of what
the reference computes.  The product path runs hand-written HIP kernels and
fails loudly when they are missing.
"""
