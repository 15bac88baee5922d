"""CPU oracle (test infrastructure only; never imported by the tokamax_amd package)."""
