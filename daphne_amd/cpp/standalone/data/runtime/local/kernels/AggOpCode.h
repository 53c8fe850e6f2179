// Stand-in for DAPHNE's src/runtime/local/kernels/AggOpCode.h:25-35: the op codes in the reference's order (the C ABI uses the same numbers).
#pragma once
enum class AggOpCode { SUM, PROD, MIN, MAX, IDXMIN, IDXMAX, MEAN, STDDEV, VAR };
