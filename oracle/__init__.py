"""ORACLE -- CPU restatements of the reference's algorithms for the hot path.
Test infrastructure only: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py, never by the distdl_amd package."""
