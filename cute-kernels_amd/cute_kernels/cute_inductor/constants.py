"""FX node kinds. Reference: cute_kernels/cute_inductor/constants.py:5-6."""

CALL_FUNCTION = "call_function"
CALL_METHOD = "call_method"
