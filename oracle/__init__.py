"""CPU oracle for the duo-causal attention path.  Test infrastructure only."""
