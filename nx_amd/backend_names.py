"""Callback names in the numeric order of the op codes in include/hipnx.h."""
BINARY_OPS = ["add", "subtract", "multiply", "divide", "pow", "remainder", "atan2", "min", "max", "quotient",
              "bitwise_and", "bitwise_or", "bitwise_xor", "left_shift", "right_shift", "equal", "not_equal",
              "greater", "less", "greater_equal", "less_equal", "logical_and", "logical_or", "logical_xor"]
UNARY_OPS = ["exp", "expm1", "log", "log1p", "sigmoid", "cos", "sin", "tan", "cosh", "sinh", "tanh", "acos", "asin",
             "atan", "acosh", "asinh", "atanh", "sqrt", "rsqrt", "cbrt", "erf", "erfc", "erf_inv", "abs",
             "bitwise_not", "ceil", "floor", "negate", "round", "sign", "count_leading_zeros", "population_count",
             "is_nan", "is_infinity"]
