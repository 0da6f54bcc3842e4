"""CPU oracle for the SRU elementwise recurrence: test infrastructure only.

Only the tests, the smoke check and the CPU-baseline leg of the benchmark may
import this package; the shipped path never does.
"""
