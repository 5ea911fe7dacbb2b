"""CPU oracle for the decode hot path — test infrastructure, not product code."""
