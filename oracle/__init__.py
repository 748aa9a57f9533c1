"""CPU oracle (test infrastructure only): C restatement of the reference's cpu_ref path."""
