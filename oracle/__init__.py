"""CPU oracle for the executor's data path — test infrastructure, never part of the product."""
