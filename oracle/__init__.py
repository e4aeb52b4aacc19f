"""CPU oracle for the fused MoE forward path -- TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this package; the product
library never does.  `binding` wraps `liboracle.so` (built from `moe_oracle.c` by the Makefile here).
"""
