"""CPU oracle for the int4 decode linears: test infrastructure, never shipped code."""
