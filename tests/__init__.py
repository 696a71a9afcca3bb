"""Parity tests: the oracle against the reference's own checks (CPU) and the HIP library against the oracle (GPU)."""
