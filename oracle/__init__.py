"""CPU checkers for the attention hot path.

TEST INFRASTRUCTURE ONLY: importable from tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg.  The shipped package (mycaffe_amd) never imports
this directory.
"""
