// Stand-in for DAPHNE's src/runtime/local/kernels/BinaryOpCode.h:29-55: the op codes in the reference's order (the C ABI uses the same numbers).
#pragma once
enum class BinaryOpCode { ADD, SUB, MUL, DIV, POW, MOD, LOG, EQ, NEQ, LT, LE, GT, GE, MIN, MAX, AND, OR, BITWISE_AND, CONCAT };
