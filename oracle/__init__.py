"""CPU oracle for the SLAYER temporal kernels: test infrastructure only (see oracle.py)."""
