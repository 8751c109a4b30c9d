"""CPU oracle package -- test infrastructure only (see vi_oracle.c header).

Importable from tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg;
never from the shipped `verinf_amd` package.
"""
