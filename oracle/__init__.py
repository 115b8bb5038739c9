"""CPU oracle (test infrastructure only; never imported by convlogic_amd)."""
