"""TEST INFRASTRUCTURE ONLY.  Eager-Aten oracle and seeded inputs for the mi355x
hot path; see oracle/eager.py.  Nothing in the product package imports this."""
