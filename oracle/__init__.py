"""TEST INFRASTRUCTURE ONLY — CPU restatement of the reference's MoE path.
Imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg;
never by the product package."""
