"""CPU checker for the aggregation path: TEST INFRASTRUCTURE ONLY.

Imported by ``tests/``, by the smoke check and by the benchmark's
``cpu_baseline`` leg; never by the shipped package.  ``c_oracle`` wraps the C
restatement in ``eppgcn_oracle.c``; ``closed_forms`` holds independent numpy
closed forms of the same functions.
"""
