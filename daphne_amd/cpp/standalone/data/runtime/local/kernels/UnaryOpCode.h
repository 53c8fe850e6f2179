// Stand-in for DAPHNE's src/runtime/local/kernels/UnaryOpCode.h:28-55: the op codes in the reference's order (the C ABI uses the same numbers).
#pragma once
enum class UnaryOpCode { MINUS, ABS, SIGN, SQRT, EXP, LN, SIN, COS, TAN, ASIN, ACOS, ATAN, SINH, COSH, TANH, FLOOR, CEIL, ROUND, ISNAN, UPPER, LOWER };
