"""CPU oracle for the LuxLib fused-operator path.  TEST INFRASTRUCTURE ONLY: imported by
tests, the smoke check and the benchmark's cpu_baseline leg; never by the product path."""
