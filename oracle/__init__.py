"""CPU oracle for the MoE grouped-GEMM path. Test infrastructure only: imported by tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the applied_ai_amd package."""
