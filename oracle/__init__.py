"""CPU oracle of the paged-KV attention path: test infrastructure only (see oracle.py)."""
