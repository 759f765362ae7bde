"""CPU oracle for the fused quantized decode path.  Test infrastructure only:
imported by tests/, the smoke check and the cpu_baseline leg of bench.py."""
