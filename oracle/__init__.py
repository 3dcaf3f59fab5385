"""Checkers for the tests and the benchmark's baseline legs.  TEST INFRASTRUCTURE ONLY: nothing in gpuk_amd imports this
package.  torch_oracle.py / gpuk_oracle.c restate the reference's torch code on the CPU; ref_kernels.py loads the
reference's own GPU kernels where oracle/_ref was built from a checkout of the reference."""
