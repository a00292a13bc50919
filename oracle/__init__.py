"""CPU oracle of the gated-MLP hot path.  TEST INFRASTRUCTURE ONLY: imported by tests/, by
__graft_entry__.smoke() and by the cpu_baseline leg of bench.py as the checker; never by the
triton_gated_mlp package."""
