"""CPU oracle of the FP8 flash-attention forward pipeline.  TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check of __graft_entry__.py and the cpu_baseline leg of bench.py may import
this package, and only as the checker; the product (cutlass_flash_atten_fp8_amd) never does.
"""
