"""CPU oracle for the grilly transformer-forward path: TEST INFRASTRUCTURE ONLY.

Nothing under grilly_amd/ may import this package; tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py are its only users."""
