"""CPU oracle for the RG-LRU path: test infrastructure only, never a product code path."""
