"""CPU oracle for the tree-attention decode path.

TEST INFRASTRUCTURE ONLY. Nothing in the shipped package imports this directory;
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may use it,
and only as the checker, never as the thing that is measured or shipped.
"""
