"""CPU oracle for the MLA flash_attn_ext path.  TEST INFRASTRUCTURE ONLY: imported by tests/, bench.py's
cpu_baseline leg and __graft_entry__.smoke() as the checker; never by jittorinfer_amd."""
