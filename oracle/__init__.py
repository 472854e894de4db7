"""CPU oracle for the attention-JVP path: test infrastructure, never imported by the product."""
