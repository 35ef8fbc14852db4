"""CPU oracle (test infrastructure only; the shipped library never imports this package)."""
