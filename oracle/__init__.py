"""
CPU oracle of the k-means Lloyd path.  TEST INFRASTRUCTURE ONLY: imported by tests/, by
__graft_entry__.smoke() and by the cpu_baseline leg of bench.py -- never by heat_amd.
"""
