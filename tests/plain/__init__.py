"""Plain, slow, whole-sequence implementation of the Llama decoder used as the oracle.

Nothing in this package imports from ``libllm_amd``: it has its own file reader, its own
configuration handling and its own arithmetic (numpy, float64 by default).
"""
