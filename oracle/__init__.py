"""CPU oracle for the attention path: test infrastructure only, never imported by the product."""
