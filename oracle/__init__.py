"""CPU oracle package (test infrastructure only; never imported by gorgonia_amd)."""
