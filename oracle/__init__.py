"""CPU oracle for the fused normalisation path: test infrastructure, never shipped."""
