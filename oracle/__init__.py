"""CPU oracle for the fused norm ops: test infrastructure, never the product path."""
