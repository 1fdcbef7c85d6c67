# Format bit flags, same values as the reference (python/gs/format.py:1-3).
_COO = 1
_CSC = 2
_CSR = 4
