"""CPU oracle for the sparse MoE block: TEST INFRASTRUCTURE ONLY.

``oracle.binding`` loads ``oracle/libmoe_oracle.so`` (built from ``moe_oracle.c`` by
``oracle/Makefile``) through ctypes.  Only the tests, the smoke check and the benchmark's
``cpu_baseline`` leg import this package; the shipped library never does.
"""
