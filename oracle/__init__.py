"""CPU oracle for the Linear4bit forward path: test infrastructure, not product code."""
