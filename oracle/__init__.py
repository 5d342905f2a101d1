"""CPU oracle for the mixed INT4/FP6 GEMM path.  Test infrastructure only."""
