"""TEST INFRASTRUCTURE ONLY: CPU oracle for the hot path.  Nothing under torpor_amd/ may
import this package; it is used by tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg."""
