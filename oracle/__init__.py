"""CPU oracles for the varlen depthwise conv -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this package;
nothing under nanoplm_amd/ does.
"""
