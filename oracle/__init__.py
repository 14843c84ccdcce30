"""CPU oracle (test infrastructure only; never imported by qtip_amd)."""
