"""CPU oracle (test infrastructure).  Never imported by the shipped package."""
