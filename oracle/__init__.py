"""CPU restatement of the reference's retrieval path: test infrastructure only."""
