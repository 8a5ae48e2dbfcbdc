"""CPU oracle for the hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under piper_amd/ may import this package.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py use it, and only as the checker / the timed CPU baseline.

It restates, in plain PyTorch-CPU / numpy, the algorithm of the reference's expert region and
bucket path; every function cites the reference lines it follows.  No reference code is imported.
"""
