"""Test-only checkers for the ternary sparse GEMM path (CPU oracle and CPU baselines).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
package; the shipped library (ternaryllm_amd) never does.
"""
