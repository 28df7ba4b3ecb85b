"""TEST INFRASTRUCTURE: CPU restatement of the reference's MoE forward (see moe_ref.c).

Only tests/, the smoke check and bench.py's cpu_baseline leg import this package."""
