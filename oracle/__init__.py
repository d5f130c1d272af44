"""CPU oracle for the mixture-of-experts forward path: test infrastructure only."""
