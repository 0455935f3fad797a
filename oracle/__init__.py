"""CPU oracle -- TEST INFRASTRUCTURE, not product code.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may
import this package; the hip backend never does.  See oracle/nervanacpu.py for
what each function restates and what pins it.
"""
