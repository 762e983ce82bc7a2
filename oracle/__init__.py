"""Test infrastructure only: CPU oracle of the quantized-linear path (see qf_oracle.c)."""
