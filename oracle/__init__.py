"""CPU checker for the moderngpu hot path.  Test infrastructure only."""
