"""CPU oracle for the dense tensor kernels: test infrastructure, not product code."""
