"""CPU oracle (test infrastructure): NumPy restatement + C restatement of the reference path."""
