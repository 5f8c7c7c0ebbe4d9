"""CPU oracle for the fp8 / int4 op family: test infrastructure only.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import this package.  The product (gaudi-pytorch-bridge_amd/) never does.
"""
