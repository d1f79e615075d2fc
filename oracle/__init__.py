"""CPU oracle of the PTv3 forward hot path.

TEST INFRASTRUCTURE. Importable only from tests/, from __graft_entry__.smoke() and from
the cpu_baseline leg of bench.py — never from the shipped package, which must fail when
its HIP library is missing instead of computing anything on the CPU.
"""
