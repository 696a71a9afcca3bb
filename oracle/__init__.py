"""CPU restatement of the reference ops: test infrastructure, never imported by the package."""
