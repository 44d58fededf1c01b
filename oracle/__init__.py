"""CPU oracle (test infrastructure only; never imported by ``steptronoss_amd``)."""
