"""CPU restatement of the reference's elementwise + reduction semantics.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py as the checker / the timed CPU baseline.  Nothing under
dpnp_amd/ imports it and no product path may call it.
"""
