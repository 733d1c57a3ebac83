"""Test oracle: CPU restatement of Axiom's CPU algorithms.  TEST INFRASTRUCTURE
ONLY -- nothing in axiom_amd imports this package."""
